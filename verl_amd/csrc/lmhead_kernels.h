// LM head fused with the row reduction: logits[tok][v] = sum_k H[tok][k] * W[v][k] are formed on the matrix cores
// and folded straight into the online-softmax partial (m, s, t) of their token; they never reach HBM.
//
// lmhead_partial_kernel: one workgroup of 8 wavefronts (two per SIMD) owns 256 tokens and walks a range of 256-row
// vocabulary tiles (its "split"); per tile it runs the full contraction in steps of 64 (v_mfma_f32_16x16x32 on
// bf16 / fp16, fp32 accumulators: with operands whose bits toggle like real data the power-managed part sustains a
// higher clock on this instruction than on 32x32x16). A wavefront owns a 64 (vocabulary) x 128 (tokens) part of the
// tile: 4 x 8 blocks of 16x16 = 128 accumulator registers, so two wavefronts fit a SIMD and one's matrix instructions
// cover the other's waits. Operands go global -> LDS directly (128-bit loads) into a ring of five 32 KiB operand tiles
// (all 160 KiB of a CU's LDS, one workgroup per CU), swizzled so that the 128-bit fragment reads are free of bank
// conflicts (measured: SQ_LDS_BANK_CONFLICT = 0). A step is two halves of 32 contraction elements with one workgroup
// barrier between them; the loads of the tiles two steps ahead are spread over the step and issued by one wavefront of
// each SIMD only, so that its partner always has matrix instructions to issue (lm_walk_tiles).
// The MFMA is issued with the vocabulary on its row side so that a lane's 4 results of a block are 4 consecutive
// vocabulary entries of ONE token: the softmax state needs no cross-lane traffic until the very end, and a gradient
// or product block is one 8-byte store.
//
// lmhead_dlogits_kernel: the same walk over (token block, vocabulary tiles) for the backward pass. The logits tile is
// recomputed on the matrix cores and turned, in registers, into the gradient with respect to the logits
// (the row-backward arithmetic of backward_kernels.h), which is stored in the operands' type.
//
// lm_gemm_kernel: out (+)= Y . X^T on the same walk, for the two products that follow (d hidden, d W).
//
// lmhead_finish_kernel: one wavefront per token forms the label's logit as a dot product in fp32, merges the
// token's partial states and writes log-prob, entropy and logsumexp (same finish as the row kernel).
//
// Roofline: dense bf16 MFMA. 2 * tokens * vocab * hidden flops; HBM traffic is the weight once per XCD group.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "backward_kernels.h"
#include "rowscore_kernels.h"

namespace vrl {

#define VRL_LDS_AS __attribute__((address_space(3)))
#define VRL_GLOBAL_AS __attribute__((address_space(1)))

typedef float lm_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kLmTokens = 256;                    // tokens per workgroup tile
constexpr int kLmVocab = 256;                     // vocabulary rows per tile
constexpr int kLmK = 64;                          // contraction elements per step: 128 bytes per tile row, whole cache lines
constexpr int kLmRowBytes = kLmK * 2;
constexpr int kLmTileBytes = 256 * kLmRowBytes;   // one operand tile in LDS (32 KiB)
constexpr int kLmRingSlots = 5;                   // operand tiles resident in LDS
constexpr int kLmLdsBytes = kLmRingSlots * kLmTileBytes;   // 160 KiB: all of a CU's LDS
constexpr int kLmMaxSplits = 64;
// The forward kernel hands over a token's softmax state once per kLmSubTiles vocabulary tiles (and wavefront quarter)
// instead of once per workgroup: what is summed in which order then depends on the vocabulary alone, not on how its
// tiles are dealt to workgroups, so a token's results are the same bits whatever the number of tokens or splits of the
// call. A workgroup's share of the vocabulary is a whole number of such runs.
constexpr int kLmSubTiles = 3;

template <int DT>
struct LmFrag;
template <>
struct LmFrag<1> {
  typedef __bf16 type __attribute__((ext_vector_type(8)));
  __device__ static __forceinline__ lm_f32x4 mfma16(type a, type b, lm_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct LmFrag<2> {
  typedef _Float16 type __attribute__((ext_vector_type(8)));
  __device__ static __forceinline__ lm_f32x4 mfma16(type a, type b, lm_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

constexpr int kLmWaves = 8;                       // wavefronts per workgroup: 4 vocabulary quarters x 2 token halves

// Which (token block, vocabulary split) a workgroup serves. Hardware deals workgroups round-robin over the 8 XCDs
// (id % 8) and each XCD starts its share in id order, 32 at a time (one per CU: the kernels take a CU's LDS). Two
// things follow. Every XCD must get the same number of workgroups that have work, or the launch waits for the fullest
// one (a grid with idle ids spread through it took up to twice as long). And the 32 that are resident on one XCD
// together should share operands through its L2. So the pairs are put in one order in which neighbours share - 8
// splits of one token block, then of the next block, ... then the next 8 splits - and that order is dealt 32
// consecutive pairs (4 token blocks x 8 splits) to an XCD at a time; what is left after the last whole round of 256 is
// cut into 8 equal runs. Only ids at the very end of the grid are idle (split < 0), and such a workgroup returns before
// any barrier. (Other shapes of 32 - 8 x 4, 16 x 2, 32 x 1 - measured the same to 3 % slower.)
constexpr int kXcds = 8;
constexpr int kXcdCus = 32;

struct LmWork {
  int split;         // < 0: nothing to do
  int64_t tok0;      // first token of the block
  int64_t tok0_ld;   // first token of the 256 rows that are loaded (an edge block is moved back so all rows exist)
  int64_t vt_begin;  // vocabulary tiles [vt_begin, vt_end)
  int64_t vt_end;
};

// Workgroups to launch for n_pairs (token block, split) pairs; the host and the kernels agree through this.
__host__ __device__ inline int64_t lm_dealt_grid(int64_t n_pairs) {
  const int64_t round = kXcds * kXcdCus;
  const int64_t full = (n_pairs / round) * round;
  return full + (n_pairs - full + kXcds - 1) / kXcds * kXcds;
}

// Position of workgroup `id` in the shared order, or -1.
__device__ __forceinline__ int64_t lm_dealt_position(int64_t id, int64_t n_pairs) {
  const int64_t round = kXcds * kXcdCus;
  const int64_t full = (n_pairs / round) * round;
  const int x = (int)(id & (kXcds - 1));
  if (id < full) {
    const int64_t local = id / kXcds;
    return ((local / kXcdCus) * kXcds + x) * kXcdCus + local % kXcdCus;
  }
  const int64_t per = (n_pairs - full + kXcds - 1) / kXcds;
  const int64_t k = full + x * per + (id - full) / kXcds;
  return k < n_pairs ? k : -1;
}

constexpr int kLmDealSplits = 8;

__device__ __forceinline__ LmWork lm_work(int64_t V, int64_t T, int n_splits, int tiles_per_split) {
  LmWork w;
  const int64_t tblocks = (T + kLmTokens - 1) / kLmTokens;
  const int64_t k = lm_dealt_position(blockIdx.x, tblocks * n_splits);
  // columns of kLmDealSplits splits (the last one narrower), one after another; in a column, token block by token block
  const int64_t col = k / (tblocks * kLmDealSplits);
  const int64_t in_col = k - col * tblocks * kLmDealSplits;
  const int rest = n_splits - (int)col * kLmDealSplits;
  const int width = rest < kLmDealSplits ? rest : kLmDealSplits;
  const int64_t tb = in_col / width;
  w.split = k < 0 ? -1 : (int)(col * kLmDealSplits + in_col % width);
  w.tok0 = tb * kLmTokens;
  w.tok0_ld = w.tok0 + kLmTokens <= T ? w.tok0 : T - kLmTokens;
  const int64_t n_vtiles = (V + kLmVocab - 1) / kLmVocab;
  w.vt_begin = (int64_t)w.split * tiles_per_split;
  w.vt_end = w.vt_begin + tiles_per_split;
  if (w.vt_end > n_vtiles) w.vt_end = n_vtiles;
  return w;
}

// The matrix-core walk shared by the forward and backward kernels. All 512 threads call it. For every vocabulary
// tile of `work` it forms the 256 x 256 block of logits of tokens [tok0_ld, tok0_ld + 256) and hands this wavefront's
// 64 (vocabulary) x 128 (tokens) part to on_tile(vt, acc): acc[i][j][v] (i < 4, j < 8, v < 4) is the logit of
//   vocabulary row  tile_row0 + wv*64 + i*16 + 4*(lane>>4) + v
//   token           tok0_ld + wt*128 + j*16 + (lane&15)
// with wv = wave>>1, wt = wave&1 and tile_row0 = vt*256 (V-256 for an edge tile, whose rows below vt*256 repeat the
// tile before). `lds` is kLmLdsBytes (160 KiB), 1 KiB aligned. On return no load is in flight; callers that reuse
// `lds` afterwards put a workgroup barrier first.
//
// LDS is a ring of five 32 KiB operand tiles. Item 2s is the W tile of global step s (a step = 64 contraction elements
// of one vocabulary tile), item 2s+1 its H tile; item n lives in slot n mod 5. A step is two halves of 32 contraction
// elements, 32 matrix instructions each, with ONE set of fragments (4 of W, 8 of H): the products run column by column,
// an H fragment is dead after its 4 products and a W fragment after the last column, and each is refilled in place with
// the next half's as soon as it is dead - the second half's from this step's tiles during the first half, the next
// step's first half from the next tiles during the second. During step s:
//   first half    requests W(s+2) into the slot H(s-1) left (eight loads per loading wavefront)
//   barrier       the step's only one: every wavefront holds the second half's fragments, so W(s) and H(s) are dead,
//                 and W(s+1), H(s+1) have landed (vmcnt(8): only the eight W(s+2) loads may still be in flight)
//   second half   requests H(s+2) into the slot W(s) left
// so the 64 loads a step needs are spread over it instead of arriving at the address unit in one burst, and the W tile
// (the operand that comes from HBM) has a step and a half to land. Every matrix instruction is followed by at most one
// fragment read and one load; the scheduling-group barriers pin that interleave (left alone, the compiler gathers the
// reads in front of the barrier, where all eight wavefronts then wait for them together).
// Only wavefronts 0-3 load (LOADER), one per SIMD: a load instruction holds its wavefront in issue for tens of cycles
// while the address unit takes it, and when both wavefronts of a SIMD carry loads at the same places of the same
// instruction stream they are held at the same time and the SIMD's matrix pipe idles. With one loading and one purely
// computing wavefront per SIMD the pipe always has a wavefront to issue from: 6.11 against 6.49 ms for the forward at
// 8192 x 3584 -> 152064 bf16 in one process, with the very same results. The two roles are two instantiations of the
// walk, chosen by a wave-uniform branch, so each stays straight-line code.
// EPILOGUE_STORES != 0: on_tile writes to global memory. Stores count in vmcnt like loads but complete in their own order.
//   1: the first barrier after on_tile waits for everything (loads and stores).
//   2: a loading wavefront still waits only until at most its eight newest loads are in flight. Loads complete in the order
//      they were issued, so once no more than eight operations are outstanding every older load has landed, whatever stores
//      the epilogue put between them (a store that is still in flight only makes the wait longer, never shorter); a
//      computing wavefront has no loads to wait for and leaves its stores to drain behind the next tile.
// Which of the two is faster differs by kernel (1-1.5 % either way, measured per kernel in one process).
//
// W_CM / H_CM: that operand is stored contraction-major, M[k][row] with `stride` elements between consecutive k (the
// layout of the other factor of a product whose contraction runs over the operands' rows, e.g. W itself in G . W).
// A tile is then 64 rows of k x 512 bytes; one wave instruction still moves 8 memory rows x 128 bytes (8 k x 64 rows).
// In LDS the tile is [k>>3][16-row block][k&7 (^4 for odd k>>3)][16 rows]: a fragment is two transposing reads
// (ds_read_b64_tr_b16: 16 lanes read 4 k x 16 rows and each receives the 4 k of its row), the 8 k-rows a half
// wavefront reads fall on distinct banks, and the row block enters the address as a plain offset of 256 bytes.
template <int DT, int EPILOGUE_STORES, bool W_CM, bool H_CM, int LOAD_GROUP, int LOAD_PHASE, int H_DELAY, bool LOADER,
          class OnTile>
__device__ __forceinline__ void lm_walk_tiles_as(const uint16_t* __restrict__ W, const uint16_t* __restrict__ H, int64_t V,
                                                 int64_t K, int64_t w_stride, int64_t h_stride, const LmWork& work,
                                                 char* lds, OnTile&& on_tile) {
  using FragT = typename LmFrag<DT>::type;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: keeps tile addressing in scalar registers
  const int wv = wave >> 1;  // vocabulary quarter of the tile
  const int wt = wave & 1;   // token half of the tile
  const int ksteps = (int)(K / kLmK);

  // Loading wavefront p = wave & 3 brings rows [64p, 64p + 64) of a tile (contraction rows [16p, 16p + 16) of a
  // contraction-major one) with eight instructions.
  // One wave instruction moves 8 tile rows x 128 bytes into LDS (lane l lands at byte l*16 of the 1 KiB block): lane l
  // serves row r = l>>3 of the block and physical 16-byte slot p = l&7, and fetches the logical chunk that the swizzle
  // assigns to that slot. Physical slot p of tile row R holds logical chunk p ^ ((R >> 1) & 7): 16 consecutive rows
  // then cover 16 distinct (row parity, slot) pairs, i.e. all 64 banks once per 16 lanes of a 128-bit read. Blocks of
  // 8 rows alternate in the swizzle's row bits, hence two lane offsets.
  const int lr = lane >> 3;
  const int lc_e = (lane & 7) ^ (lr >> 1), lc_o = (lane & 7) ^ (4 + (lr >> 1));
  // contraction-major: lane l lands in (block l>>4 of the instruction's four, k&7 slot (l&15)>>1, 16-byte half l&1) and
  // fetches memory row (slot, ^4 in an odd group of 8 contraction rows) of the group's eight, bytes 32*(l>>4) + 16*(l&1)
  // of the 128. A loading wavefront's instructions 0-3 serve its even group, 4-7 its odd one.
  const int cm_slot = (lane & 15) >> 1;
  const int cm_byte = (lane >> 4) * 32 + (lane & 1) * 16;
  const uint32_t w_lane_e = W_CM ? (uint32_t)(cm_slot * w_stride * 2 + cm_byte) : (uint32_t)((lr * w_stride + lc_e * 8) * 2);
  const uint32_t w_lane_o = W_CM ? (uint32_t)((cm_slot ^ 4) * w_stride * 2 + cm_byte) : (uint32_t)((lr * w_stride + lc_o * 8) * 2);
  const uint32_t h_lane_e = H_CM ? (uint32_t)(cm_slot * h_stride * 2 + cm_byte) : (uint32_t)((lr * h_stride + lc_e * 8) * 2);
  const uint32_t h_lane_o = H_CM ? (uint32_t)((cm_slot ^ 4) * h_stride * 2 + cm_byte) : (uint32_t)((lr * h_stride + lc_o * 8) * 2);
  // bytes of 8 memory rows, from one step to the next (64 contraction elements), and from tile row 0 to the
  // wavefront's first memory row
  const uint64_t w_blk = (uint64_t)(8 * w_stride * 2);
  const uint64_t h_blk = (uint64_t)(8 * h_stride * 2);
  const uint64_t w_adv = W_CM ? (uint64_t)(kLmK * w_stride * 2) : (uint64_t)kLmRowBytes;
  const uint64_t h_adv = H_CM ? (uint64_t)(kLmK * h_stride * 2) : (uint64_t)kLmRowBytes;
  const uint64_t w_row = W_CM ? (uint64_t)2 : (uint64_t)(w_stride * 2);   // bytes per tile row
  const uint64_t h_row = H_CM ? (uint64_t)2 : (uint64_t)(h_stride * 2);
  const int pw = wave & 3;
  const uint64_t w_first = (uint64_t)pw * (W_CM ? 2 : 8) * w_blk;
  const uint64_t h_first = (uint64_t)pw * (H_CM ? 2 : 8) * h_blk;

  // Two load cursors, one per operand: uniform byte pointers to this wavefront's first row of the W / H tile to
  // request next, and the ring slot it goes to. A step advances a pointer by 64
  // contraction elements; at the end of a vocabulary tile W jumps to the next tile's rows and H returns to k = 0. Past
  // the last step the pointers stay put: the last tiles are requested again into slots nobody reads any more (in
  // bounds, harmless), so the main loop needs no "is there more" branch around its loads.
  const int64_t total_steps = (work.vt_end > work.vt_begin ? (work.vt_end - work.vt_begin) : 0) * ksteps;
  auto uniform64 = [](uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  auto vrow_of = [&](int64_t vt) { return (vt + 1) * kLmVocab <= V ? vt * kLmVocab : V - kLmVocab; };
  uint64_t wp = uniform64(reinterpret_cast<uint64_t>(W) + (uint64_t)vrow_of(work.vt_begin) * w_row + w_first);
  uint64_t hp = uniform64(reinterpret_cast<uint64_t>(H) + (uint64_t)work.tok0_ld * h_row + h_first);
  int64_t w_step = 0, w_vt = work.vt_begin, h_step = 0;
  int w_ks = 0, h_ks = 0;
  int w_slot = 0, h_slot = 1;
  const int wave_rows = pw * 64 * kLmRowBytes;
  // instruction i of eight: rows 8i .. 8i+7 of the wavefront's 64; contraction-major: group i>>2 of its two groups of
  // 8 contraction rows, rows 64*(i&3) .. +63 of the tile (128 bytes of each memory row)
  auto load_w = [&](int i) {
    const char* src = reinterpret_cast<const char*>(wp + (W_CM ? (i >> 2) * w_blk + (i & 3) * 128 : i * w_blk));
    const bool odd = W_CM ? ((i >> 2) & 1) : (i & 1);
    __builtin_amdgcn_global_load_lds((const VRL_GLOBAL_AS void*)(src + (odd ? w_lane_o : w_lane_e)),
                                     (VRL_LDS_AS void*)(lds + w_slot * kLmTileBytes + wave_rows + i * 8 * kLmRowBytes), 16, 0, 0);
  };
  auto load_h = [&](int i) {
    const char* src = reinterpret_cast<const char*>(hp + (H_CM ? (i >> 2) * h_blk + (i & 3) * 128 : i * h_blk));
    const bool odd = H_CM ? ((i >> 2) & 1) : (i & 1);
    __builtin_amdgcn_global_load_lds((const VRL_GLOBAL_AS void*)(src + (odd ? h_lane_o : h_lane_e)),
                                     (VRL_LDS_AS void*)(lds + h_slot * kLmTileBytes + wave_rows + i * 8 * kLmRowBytes), 16, 0, 0);
  };
  auto next_slot = [](int slot) { return slot + 2 >= kLmRingSlots ? slot + 2 - kLmRingSlots : slot + 2; };
  // (branch-free: the quarter steps of a step stay one basic block, which lets the compiler count outstanding LDS
  // reads exactly instead of waiting for all of them at every block boundary)
  auto advance_w = [&]() {
    w_slot = next_slot(w_slot);
    const bool more = w_step + 1 < total_steps;
    const bool tile_end = w_ks + 1 == ksteps;
    const int64_t dv = vrow_of(w_vt + 1) - vrow_of(w_vt);
    const uint64_t jump = (uint64_t)dv * w_row - (uint64_t)(ksteps - 1) * w_adv;
    wp += more ? (tile_end ? jump : w_adv) : (uint64_t)0;
    w_vt += (more && tile_end) ? 1 : 0;
    w_ks = more ? (tile_end ? 0 : w_ks + 1) : w_ks;
    ++w_step;
  };
  auto advance_h = [&]() {
    h_slot = next_slot(h_slot);
    const bool more = h_step + 1 < total_steps;
    const bool tile_end = h_ks + 1 == ksteps;
    const uint64_t back = (uint64_t)0 - (uint64_t)(ksteps - 1) * h_adv;
    hp += more ? (tile_end ? back : h_adv) : (uint64_t)0;
    h_ks = more ? (tile_end ? 0 : h_ks + 1) : h_ks;
    ++h_step;
  };

  // Fragment addresses. Row-major tile: row (within its 16-row block) = lane&15, logical chunk = 4*half + (lane>>4).
  // Contraction-major tile: the lane's group g = lane>>4 owns k = 32*half + 8*g .. +7 and fetches them with two
  // transposing reads (k .. k+3 and k+4 .. k+7); in each, lane s = lane&15 of the group supplies the address of
  // k-row s>>2, rows 4*(s&3) .. +3 of the block.
  int phys[2], cm_q[2];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    phys[hf] = (((4 * hf + (lane >> 4)) ^ ((lane >> 1) & 7)) * 16);
    cm_q[hf] = (lane >> 4) * 4096 + (4 * (hf ^ ((lane >> 4) & 1)) + ((lane & 15) >> 2)) * 32 + (lane & 3) * 8;
  }
  constexpr int kWBlock = W_CM ? 256 : 16 * kLmRowBytes;   // from one 16-row block of a tile to the next
  constexpr int kHBlock = H_CM ? 256 : 16 * kLmRowBytes;
  constexpr int kCmHalf = 4 * 4096;                         // second half of a contraction-major tile
  const int fragoff_w = W_CM ? wv * 4 * 256 : (wv * 64 + (lane & 15)) * kLmRowBytes;    // within a W slot
  const int fragoff_h = H_CM ? wt * 8 * 256 : (wt * 128 + (lane & 15)) * kLmRowBytes;   // within an H slot
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  auto read_cm = [](const char* p0, const char* p1) {
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((VRL_LDS_AS s16x4*)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((VRL_LDS_AS s16x4*)p1);
    const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(FragT, v);
  };
  // p0 (and p1 for a contraction-major tile) point at block 0 of the wanted half of a slot
  auto read_w = [&](const char* p0, const char* p1, int i) {
    if constexpr (W_CM) return read_cm(p0 + i * kWBlock, p1 + i * kWBlock);
    else return *reinterpret_cast<const FragT*>(p0 + i * kWBlock);
  };
  auto read_h = [&](const char* p0, const char* p1, int j) {
    if constexpr (H_CM) return read_cm(p0 + j * kHBlock, p1 + j * kHBlock);
    else return *reinterpret_cast<const FragT*>(p0 + j * kHBlock);
  };
  auto w_ptr = [&](int slot, int hf, int q) {
    return lds + slot * kLmTileBytes + fragoff_w + (W_CM ? cm_q[q] + hf * kCmHalf : phys[hf]);
  };
  auto h_ptr = [&](int slot, int hf, int q) {
    return lds + slot * kLmTileBytes + fragoff_h + (H_CM ? cm_q[q] + hf * kCmHalf : phys[hf]);
  };

  constexpr int HD = LOADER ? H_DELAY : 0;   // a loading wavefront refills an H fragment this many instructions later
  FragT a[4], b[8];
  if (total_steps > 0) {
#pragma unroll
    for (int rep = 0; rep < 2; ++rep) {
      if constexpr (LOADER) {
#pragma unroll
        for (int i = 0; i < 8; ++i) load_w(i);
      }
      advance_w();
      if constexpr (LOADER) {
#pragma unroll
        for (int i = 0; i < 8; ++i) load_h(i);
      }
      advance_h();
    }
    if constexpr (LOADER) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = read_w(w_ptr(0, 0, 0), w_ptr(0, 0, 1), i);
#pragma unroll
    for (int j = 0; j < 8; ++j) b[j] = read_h(h_ptr(1, 0, 0), h_ptr(1, 0, 1), j);
  }

  int cw = 0, ch = 1;   // ring slots of the step being computed
  bool after_epilogue = false;
  for (int64_t vt = work.vt_begin; vt < work.vt_end; ++vt) {
    lm_f32x4 acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

    for (int ks = 0; ks < ksteps; ++ks) {
      const int nw = next_slot(cw), nh = next_slot(ch);
      // Two halves of 32 contraction elements, 32 matrix instructions each, with ONE set of fragments (4 of W, 8 of H):
      // the products run column by column, an H fragment is dead after its 4 products and a W fragment after the last
      // column, and each is refilled in place with the next half's as soon as it is dead - the second half's from this
      // step's tiles during the first half, the next step's first half from the next tiles during the second. The
      // step's barrier therefore sits between the halves: behind it W(s), H(s) are dead and W(s+1), H(s+1) must have
      // landed. First half: the loading wavefronts' eight loads each of W(s+2) (into the slot H(s-1) left); second half: H(s+2)
      // (slot of W(s)).
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        if (hf == 1) {
          if (EPILOGUE_STORES == 1 && after_epilogue) {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
          } else if (LOADER) {
            asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
          } else {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          }
          __builtin_amdgcn_s_barrier();
          after_epilogue = false;
        }
        const char* rw0 = w_ptr((hf == 1) ? nw : cw, hf ^ 1, 0);
        const char* rw1 = W_CM ? w_ptr((hf == 1) ? nw : cw, hf ^ 1, 1) : rw0;
        const char* rh0 = h_ptr((hf == 1) ? nh : ch, hf ^ 1, 0);
        const char* rh1 = H_CM ? h_ptr((hf == 1) ? nh : ch, hf ^ 1, 1) : rh0;
#pragma unroll
        for (int mm = 0; mm < 32; ++mm) {
          const int j = mm >> 2, i = mm & 3;
          acc[i][j] = LmFrag<DT>::mfma16(a[i], b[j], acc[i][j]);
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            const int at = 4 * jj + 3 + HD < 31 ? 4 * jj + 3 + HD : 31;
            if (at == mm) b[jj] = read_h(rh0, rh1, jj);
          }
          if (j == 7) a[i] = read_w(rw0, rw1, i);
          if (LOADER && ((mm + 1 + LOAD_PHASE) % (4 * LOAD_GROUP)) == 0) {
#pragma unroll
            for (int q = 0; q < LOAD_GROUP; ++q) {
              const int idx = (mm + 1 + LOAD_PHASE) / 4 - 1 - q;   // 0 .. 7, each once per half
              if (hf == 0) load_w(idx); else load_h(idx);
            }
          }
        }
#pragma unroll
        for (int mm = 0; mm < 32; ++mm) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                // one matrix instruction
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            const int at = 4 * jj + 3 + HD < 31 ? 4 * jj + 3 + HD : 31;
            if (at == mm) __builtin_amdgcn_sched_group_barrier(0x100, H_CM ? 2 : 1, 0);  // an H fragment
          }
          if ((mm >> 2) == 7) __builtin_amdgcn_sched_group_barrier(0x100, W_CM ? 2 : 1, 0); // a W fragment
          if (LOADER && ((mm + 1 + LOAD_PHASE) % (4 * LOAD_GROUP)) == 0) __builtin_amdgcn_sched_group_barrier(0x010, LOAD_GROUP, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (hf == 0) advance_w(); else advance_h();
      }
      cw = nw;
      ch = nh;
    }
    on_tile(vt, acc);
    after_epilogue = true;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the last, redundant loads still target the ring
}

// LOAD_GROUP / LOAD_PHASE place the loading wavefronts' eight loads of a half: LOAD_GROUP (1 or 2) of them together
// behind every 4 * LOAD_GROUP matrix instructions, LOAD_PHASE instructions before the end of such a run (0 = behind the
// last product of a column, where the H fragment is refilled too). The kernels differ by 1-3 % in which placement suits
// them (a sweep per kernel at 8192 / 4096 x 3584 <-> 152064 bf16): the forward takes single loads at phase 0, the two
// products single loads one instruction earlier, the gradient kernel single loads three instructions earlier. H_DELAY moves the
// loading wavefronts' refills of the H fragments that many instructions back, away from the computing wavefronts' (which
// stay right behind a column's last product): worth 3 % to the d hidden product, nothing or less to the others.
template <int DT, int EPILOGUE_STORES, bool W_CM, bool H_CM, int LOAD_GROUP, int LOAD_PHASE, int H_DELAY, class OnTile>
__device__ __forceinline__ void lm_walk_tiles(const uint16_t* __restrict__ W, const uint16_t* __restrict__ H, int64_t V,
                                              int64_t K, int64_t w_stride, int64_t h_stride, const LmWork& work,
                                              char* lds, OnTile&& on_tile) {
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  if (wave < 4)
    lm_walk_tiles_as<DT, EPILOGUE_STORES, W_CM, H_CM, LOAD_GROUP, LOAD_PHASE, H_DELAY, true>(W, H, V, K, w_stride, h_stride,
                                                                                          work, lds, on_tile);
  else
    lm_walk_tiles_as<DT, EPILOGUE_STORES, W_CM, H_CM, LOAD_GROUP, LOAD_PHASE, H_DELAY, false>(W, H, V, K, w_stride, h_stride,
                                                                                           work, lds, on_tile);
}

// grid.x = token blocks * n_splits, block = 512, dynamic LDS = kLmLdsBytes. Writes, per (token, split), the online-softmax
// partial (m, s, t, 0) of the split's vocabulary tiles to partials[(token * n_splits + split) * 4 ...].
// STORE: the logits tile (the plain products, before the temperature) is also written, in the operands' type, to
// logits_out[tok * l_stride + v] (l_stride and V multiples of 8, 16-byte aligned base): what a backward pass that may
// spend memory instead of forming the logits again reads (vrl_rowscore_backward over them, in place). The softmax state
// is folded from the fp32 values all the same, so the scores do not depend on whether the logits are kept.
// The two values that meet when x is exchanged between rows of 16 lanes (round 0: row 0 with 1 and row 2 with 3; round 1:
// the lower with the upper half of the wavefront): every lane of such a pair receives the same two values, out[0] from
// the lower-numbered row(s) and out[1] from the higher.
__device__ __forceinline__ void lm_swap_rows(float x, int round, float (&out)[2]) {
  const unsigned u = __float_as_uint(x);
  if (round == 0) {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    out[0] = __uint_as_float(r[0]);
    out[1] = __uint_as_float(r[1]);
  } else {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    out[0] = __uint_as_float(r[0]);
    out[1] = __uint_as_float(r[1]);
  }
}

template <int DT, bool STORE>
__global__ __launch_bounds__(kLmWaves * 64, 1) void lmhead_partial_kernel(
    const uint16_t* __restrict__ W, const uint16_t* __restrict__ H, int64_t V, int64_t T, int64_t K, int64_t w_stride,
    int64_t h_stride, const float* __restrict__ temperature, int n_splits, int tiles_per_split,
    float* __restrict__ partials, uint16_t* __restrict__ logits_out, int64_t l_stride, int64_t l_rows) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];  // the operand ring

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wv = wave >> 1;
  const int wt = wave & 1;
  const LmWork work = lm_work(V, T, n_splits, tiles_per_split);
  if (work.split < 0) return;   // the whole workgroup: an idle slot of the grid
  const int64_t n_vtiles = (V + kLmVocab - 1) / kLmVocab;

  // per-lane softmax state for the 8 token columns this lane sees (16 x 16 blocks: column = lane & 15)
  float m[8], s[8], t[8], c[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    m[j] = neg_inf();
    s[j] = 0.f;
    t[j] = 0.f;
    const int64_t tok = work.tok0_ld + wt * 128 + j * 16 + (lane & 15);
    c[j] = make_scale<false>(temperature, tok).c;   // log2(e) / max(T, 1e-8), exactly what the finishing kernel uses
  }

  // (load placement, see lm_walk_tiles: single loads right behind a column's last matrix instruction. Pairs of loads
  // measured 2 % faster to 5 % slower from one build to the next, single loads anywhere in the column within 1 %.)
  lm_walk_tiles<DT, 2, false, false, 1, 0, 0>(W, H, V, K, w_stride, h_stride, work, lds, [&](int64_t vt, lm_f32x4 (&acc)[4][8]) {
    // fold 16 logits per token column into the running state (maximum first, then the exponentials; nothing is
    // buffered): acc[i][j][v] is vocabulary row tile_row0 + wv*64 + i*16 + 4*(lane>>4) + v of token column j
    const bool edge = (vt + 1) * kLmVocab > V;
    const int64_t vrow0 = (edge ? V - kLmVocab : vt * kLmVocab) + wv * 64 + 4 * (lane >> 4);
    const int64_t vfirst = vt * kLmVocab;   // rows below belong to the tile before
    // (the row pointer is formed per tile; the empty asm keeps it out of the main loop's registers)
    int64_t tok0v = work.tok0_ld + wt * 128 + (lane & 15);
    if constexpr (STORE) asm volatile("" : "+v"(tok0v));
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float x[16];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) x[i * 4 + v] = acc[i][j][v];
      if constexpr (STORE) {
        using O = ElemOut<DT>;
        // (false for the rows an edge block shares with the block before, and for tokens whose logits are not kept)
        if (tok0v + j * 16 >= work.tok0 && tok0v + j * 16 < l_rows) {
          uint16_t* out = logits_out + (tok0v + j * 16) * l_stride;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int64_t vr = vrow0 + i * 16;   // first of 4 consecutive vocabulary entries (a multiple of 4)
            if (vr >= vfirst) {
              uint2 pk;
              pk.x = O::pack2(x[i * 4], x[i * 4 + 1]);
              pk.y = O::pack2(x[i * 4 + 2], x[i * 4 + 3]);
              *reinterpret_cast<uint2*>(out + vr) = pk;
            }
          }
        }
      }
      if (edge) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int64_t vr = vrow0 + (e >> 2) * 16 + (e & 3);
          x[e] = vr >= vfirst ? x[e] : neg_inf();
        }
      }
      float bm = neg_inf();
#pragma unroll
      for (int e = 0; e < 16; ++e) bm = __builtin_fmaxf(bm, x[e]);
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
      for (int e = 0; e < 16; ++e) {
        const float d = __builtin_fmaf(x[e], c[j], -sub);
        const float ex = hw_exp2(d);
        ps += ex;
        pt = __builtin_fmaf(ex, (ex == 0.f) ? 0.f : d, pt);
      }
      s[j] += ps;
      t[j] += pt;
      // one token column at a time: keeps the compiler from pulling the next columns' accumulator copies forward
      __builtin_amdgcn_sched_barrier(0);
    }
    // End of a run of kLmSubTiles tiles (or of the vocabulary): hand the state over and start afresh. Lanes l, l^16,
    // l^32, l^48 hold the same tokens (other vocabulary rows): they are combined here, the four vocabulary-quarter
    // wavefronts and the runs by the finishing kernel. partials[(token * n_runs * 4 + run * 4 + quarter) * 3 + {m, s, t}]:
    // a token's states lie together for the finishing kernel; here a lane stores 12 bytes per token column.
    if ((vt + 1) % kLmSubTiles == 0 || vt + 1 == n_vtiles) {
      const int64_t n_states = ((n_vtiles + kLmSubTiles - 1) / kLmSubTiles) * 4;
      const int64_t tok_lane = work.tok0_ld + wt * 128 + (lane & 15);
      float* dst = partials + (tok_lane * n_states + (vt / kLmSubTiles) * 4 + wv) * 3;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float M = m[j], S = s[j], Tt = t[j];
        // rows of 16 lanes pairwise (0 with 1, 2 with 3), then the two halves of the wavefront: the swaps are vector-ALU
        // instructions (an exchange through the LDS crossbar would wait behind the ring's fragment reads), and every
        // lane of a pair computes the same merge of the same two states
#pragma unroll
        for (int round = 0; round < 2; ++round) {
          float pm[2], ps[2], pt[2];
          lm_swap_rows(M, round, pm);
          lm_swap_rows(S, round, ps);
          lm_swap_rows(Tt, round, pt);
          const float N = __builtin_fmaxf(pm[0], pm[1]);
          float S2 = 0.f, T2 = 0.f;
          if (N != neg_inf()) {
            const float a1 = hw_exp2(pm[0] - N), a2 = hw_exp2(pm[1] - N);
            const float d1 = (pm[0] == neg_inf()) ? 0.f : pm[0] - N;
            const float d2 = (pm[1] == neg_inf()) ? 0.f : pm[1] - N;
            S2 = a1 * ps[0] + a2 * ps[1];
            T2 = a1 * (pt[0] + d1 * ps[0]) + a2 * (pt[1] + d2 * ps[1]);
          }
          M = N;
          S = S2;
          Tt = T2;
        }
        // (rows that an edge block shares with the block before are that block's to write)
        if (lane < 16 && tok_lane + j * 16 >= work.tok0) {
          float* d = dst + static_cast<int64_t>(j * 16) * n_states * 3;
          d[0] = M;
          d[1] = S;
          d[2] = Tt;
        }
        m[j] = neg_inf();
        s[j] = 0.f;
        t[j] = 0.f;
      }
    }
  });
}

// Backward: dlogits[tok, v] = (g_logprob[tok] * (1[v == label[tok]] - p) - g_entropy[tok] * p * (log p + entropy[tok])) / T[tok]
// with p = exp(z - lse[tok]), z = logits / T, for all tokens and the vocabulary tiles of each split, written in the
// operands' type to dlogits[tok * d_stride + v] (d_stride, V multiples of 8; 16-byte aligned base). Same grid and LDS as
// lmhead_partial_kernel. A lane holds 4 consecutive vocabulary entries of one token per 16 x 16 block, i.e. one 8-byte
// store; lanes l, l+16, l+32, l+48 complete 32 contiguous bytes of the token's row.
template <int DT>
__global__ __launch_bounds__(kLmWaves * 64, 1) void lmhead_dlogits_kernel(
    const uint16_t* __restrict__ W, const uint16_t* __restrict__ H, int64_t V, int64_t T, int64_t K, int64_t w_stride,
    int64_t h_stride, const int64_t* __restrict__ labels, const float* __restrict__ temperature,
    const float* __restrict__ lse, const float* __restrict__ entropy, const float* __restrict__ g_logprob,
    const float* __restrict__ g_entropy, int n_splits, int tiles_per_split, uint16_t* __restrict__ dlogits,
    int64_t d_stride) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];  // the operand ring
  using O = ElemOut<DT>;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wv = wave >> 1;
  const int wt = wave & 1;
  const LmWork work = lm_work(V, T, n_splits, tiles_per_split);
  if (work.split < 0) return;   // the whole workgroup: an idle slot of the grid

  // the row constants of the 8 token columns this lane sees (16 x 16 blocks: column = lane & 15)
  RowGrad f[8];
  int label[8];       // -1: no label term
  const int64_t tok_lane0 = work.tok0_ld + wt * 128 + (lane & 15);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int64_t tok = tok_lane0 + j * 16;
    float Tm = 1.f;
    if (temperature != nullptr) {
      Tm = temperature[tok];
      Tm = (Tm < kMinTemperature) ? kMinTemperature : Tm;
    }
    const float rT = 1.0f / Tm;
    const float gl = (g_logprob != nullptr) ? g_logprob[tok] : 0.f;
    const float gh = (g_entropy != nullptr) ? g_entropy[tok] : 0.f;
    const float Hh = (g_entropy != nullptr) ? entropy[tok] : 0.f;
    f[j].c = kLog2e * rT;
    f[j].lse2 = lse[tok] * kLog2e;
    f[j].a = -(gh * kLn2f) * rT;
    f[j].b = -(gl + gh * Hh) * rT;
    f[j].lab = gl * rT;
    const int64_t lab = (g_logprob != nullptr) ? labels[tok] : -1;
    label[j] = (lab >= 0 && lab < V) ? (int)lab : -1;   // an out-of-range label was reported by the forward pass
  }

  lm_walk_tiles<DT, 2, false, false, 1, 3, 0>(W, H, V, K, w_stride, h_stride, work, lds, [&](int64_t vt, lm_f32x4 (&acc)[4][8]) {
    // acc[i][j][0..3]: vocabulary entries vr .. vr+3, vr = tile_row0 + wv*64 + i*16 + 4*(lane>>4), of token column j
    const bool edge = (vt + 1) * kLmVocab > V;
    const int vrow0 = (int)(edge ? V - kLmVocab : vt * kLmVocab) + wv * 64 + 4 * (lane >> 4);
    const int vfirst = (int)(vt * kLmVocab);   // rows below belong to the tile before
    // The row pointers are formed per tile from the first column's (the empty asm keeps loop-invariant code motion from
    // holding all 8 of them in registers through the main loop).
    int64_t tok0v = tok_lane0;
    asm volatile("" : "+v"(tok0v));
    uint16_t* out0 = dlogits + tok0v * d_stride;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool tok_mine = tok0v + j * 16 >= work.tok0;   // false for the rows an edge block shares with the block before
      uint16_t* out = out0 + (int64_t)(j * 16) * d_stride;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int vr = vrow0 + i * 16;   // first of 4 consecutive vocabulary entries (a multiple of 4)
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          y[e] = f[j](acc[i][j][e]);
          if (vr + e == label[j]) y[e] += f[j].lab;
        }
        if (tok_mine && vr >= vfirst) {
          uint2 pk;
          pk.x = O::pack2(y[0], y[1]);
          pk.y = O::pack2(y[2], y[3]);
          *reinterpret_cast<uint2*>(out + vr) = pk;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  });
}


// ---- the two products of the backward on the same walk -----------------------------------------------------------
// out[y][x] (+)= sum_k X[x][k] * Y[y][k]. An operand is either row-major, (rows, K) contiguous along k, or
// contraction-major (X_CM / Y_CM), (K, rows) contiguous along its rows, so neither product needs a transposed copy:
//   d hidden = G . W   : X = W (vocab, hidden) contraction-major, Y = G (tokens, vocab) row-major
//   d W      = G^T . H : X = H (tokens, hidden) and Y = G (tokens, vocab), both contraction-major.
// X plays the walk's vocabulary side (a lane's accumulator quad is 4 consecutive x of one y, i.e. one 8-byte
// store of out[y][x..x+3]), Y its token side.
//
// A work item is (y block of 256 rows, `tiles_per_item` x tiles, one of `k_parts` ranges of the contraction). Items
// are grouped in py x px patches of (y block, x split) pairs of one contraction range, which share their operand tiles,
// and the patches are dealt to the XCDs (see the kernel); py and px need not divide their counts, the patches at the far
// edges are smaller.
// MODE 0 stores the product in the operands' type, MODE 1 adds it to what `out` holds (one rounding, like a GEMM with
// beta = 1), MODE 2 stores fp32 partial sums at partials[(kp * NY + y) * NX + x] for lm_gemm_reduce_kernel.
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ void lm_unpack2(uint32_t w, float* x);   // two 16-bit elements of type DT -> fp32
template <>
__device__ __forceinline__ void lm_unpack2<1>(uint32_t w, float* x) {
  x[0] = __uint_as_float(w << 16);
  x[1] = __uint_as_float(w & 0xffff0000u);
}
template <>
__device__ __forceinline__ void lm_unpack2<2>(uint32_t w, float* x) { Elem<2>::unpack2(w, x); }

struct LmGemmShape {
  int64_t NX, NY;          // rows of X / of Y = columns / rows of out
  int64_t k_steps;         // contraction length / 64
  int k_parts;             // ranges the contraction is cut into
  int steps_per_part;      // ceil(k_steps / k_parts); the last range may be shorter
  int tiles_per_item;      // x tiles one workgroup walks
  int py, px;              // patch of (y blocks, x splits) per XCD
};

template <int DT, int MODE, bool X_CM, bool Y_CM>
__global__ __launch_bounds__(kLmWaves * 64, 1) void lm_gemm_kernel(
    const uint16_t* __restrict__ X, const uint16_t* __restrict__ Y, LmGemmShape g, int64_t x_stride, int64_t y_stride,
    uint16_t* __restrict__ out, int64_t out_stride, float* __restrict__ partials) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];  // the operand ring
  using O = ElemOut<DT>;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wv = wave >> 1;
  const int wt = wave & 1;

  const int64_t nyb = (g.NY + kLmTokens - 1) / kLmTokens;
  const int64_t nxt = (g.NX + kLmVocab - 1) / kLmVocab;
  const int64_t nxs = (nxt + g.tiles_per_item - 1) / g.tiles_per_item;
  // Patches of py y blocks x px x splits of one contraction range (smaller at the far edges), range by range, columns
  // of patches one after another. Whole rows of 8 patches go one patch to an XCD, whose 32 CUs then walk the contraction
  // in step on shared operand tiles; the fewer than 8 patches left at the end are dealt item by item over the XCDs
  // instead, so that every XCD ends with about the same number of items (a launch waits for the fullest one). A patch
  // has py * px slots; those past its items are idle, and such a workgroup returns before any barrier.
  const int psize = g.py * g.px;
  const int patches_y = (int)((nyb + g.py - 1) / g.py), patches_x = (int)((nxs + g.px - 1) / g.px);
  const int64_t per_part = (int64_t)patches_y * patches_x;
  const int64_t n_patches = per_part * g.k_parts;
  const int64_t dealt_whole = (n_patches / kXcds) * kXcds * psize;   // ids that take whole patches
  const int64_t id = blockIdx.x;
  int64_t patch;
  int within;
  if (id < dealt_whole) {
    const int64_t local = id / kXcds;
    patch = (local / psize) * kXcds + (id & (kXcds - 1));
    within = (int)(local % psize);
  } else {
    patch = (n_patches / kXcds) * kXcds + (id - dealt_whole) / psize;
    within = (int)((id - dealt_whole) % psize);
  }
  if (patch >= n_patches) return;   // the whole workgroup
  // (64-bit divisions run on the vector ALUs; readfirstlane brings their uniform results back to scalar registers)
  const int kp = __builtin_amdgcn_readfirstlane((int)(patch / per_part));
  const int r = __builtin_amdgcn_readfirstlane((int)(patch % per_part));
  const int row = r % patches_y, col = r / patches_y;
  const int height = (int)nyb - row * g.py < g.py ? (int)nyb - row * g.py : g.py;
  const int width = (int)nxs - col * g.px < g.px ? (int)nxs - col * g.px : g.px;
  if (within >= height * width) return;   // an idle slot of an edge patch
  const int yb = __builtin_amdgcn_readfirstlane(row * g.py + within % height);
  const int xsplit = __builtin_amdgcn_readfirstlane(col * g.px + within / height);

  LmWork work;
  work.split = kp;
  work.tok0 = (int64_t)yb * kLmTokens;
  work.tok0_ld = work.tok0 + kLmTokens <= g.NY ? work.tok0 : g.NY - kLmTokens;
  work.vt_begin = (int64_t)xsplit * g.tiles_per_item;
  work.vt_end = work.vt_begin + g.tiles_per_item;
  if (work.vt_end > nxt) work.vt_end = nxt;
  const int64_t step0 = (int64_t)kp * g.steps_per_part;
  int64_t nsteps = g.k_steps - step0;
  if (nsteps > g.steps_per_part) nsteps = g.steps_per_part;

  const uint16_t* x0 = X + step0 * kLmK * (X_CM ? x_stride : 1);
  const uint16_t* y0p = Y + step0 * kLmK * (Y_CM ? y_stride : 1);
  lm_walk_tiles<DT, 1, X_CM, Y_CM, 1, 1, (X_CM && !Y_CM) ? 1 : 0>(x0, y0p, g.NX, nsteps * kLmK, x_stride, y_stride, work, lds,
                                      [&](int64_t vt, lm_f32x4 (&acc)[4][8]) {
    // acc[i][j][0..3]: columns x0 .. x0+3 of out, x0 = tile_row0 + wv*64 + i*16 + 4*(lane>>4), of row
    // y = tok0_ld + wt*128 + j*16 + (lane&15)
    const bool edge = (vt + 1) * kLmVocab > g.NX;
    const int xrow0 = (int)(edge ? g.NX - kLmVocab : vt * kLmVocab) + wv * 64 + 4 * (lane >> 4);
    const int xfirst = (int)(vt * kLmVocab);   // columns below belong to the tile before
    // Row pointers are formed here, per tile, as "row of column block 0" + a uniform offset per block. The empty asm
    // hides the lane's row from loop-invariant code motion, which would otherwise keep all 8 pointers (16 registers)
    // alive through the main loop and spill.
    int y_lane = lane & 15;
    asm volatile("" : "+v"(y_lane));
    const int64_t y0 = work.tok0_ld + wt * 128 + y_lane;
    uint16_t* out_row0 = out + y0 * out_stride;
    float* part_row0 = partials + ((int64_t)kp * g.NY + y0) * g.NX;
    // Interior tiles (all 256 x 256 results are this item's own) store without conditions: straight-line code, whose
    // loads (MODE 1) and stores the compiler can keep in flight together. Edge tiles, which repeat rows or columns of
    // the tile before, check each quad.
    auto write_tile = [&](auto guard_tag) {
      constexpr bool GUARD = decltype(guard_tag)::value;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool y_mine = !GUARD || y0 + j * 16 >= work.tok0;
        uint16_t* out_row = out_row0 + (int64_t)(j * 16) * out_stride;
        float* part_row = part_row0 + (int64_t)(j * 16) * g.NX;
        // MODE 1: what out holds at this column's four quads, requested together (a row or column that belongs to the
        // tile before is a valid address all the same; only its store is skipped)
        uint2 old[4];
        if constexpr (MODE == 1) {
#pragma unroll
          for (int i = 0; i < 4; ++i) old[i] = *reinterpret_cast<const uint2*>(out_row + xrow0 + i * 16);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int x = xrow0 + i * 16;   // a multiple of 4
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][e];
          if constexpr (MODE == 1) {
            float o[4];
            lm_unpack2<DT>(old[i].x, o);
            lm_unpack2<DT>(old[i].y, o + 2);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += o[e];
          }
          if (!GUARD || (y_mine && x >= xfirst)) {
            if constexpr (MODE == 2) {
              f32x4 pk = {v[0], v[1], v[2], v[3]};
              *reinterpret_cast<f32x4*>(part_row + x) = pk;
            } else {
              uint2 pk;
              pk.x = O::pack2(v[0], v[1]);
              pk.y = O::pack2(v[2], v[3]);
              *reinterpret_cast<uint2*>(out_row + x) = pk;
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    if (edge || work.tok0_ld != work.tok0) write_tile(std::true_type{});
    else write_tile(std::false_type{});
  });
}

// out[y][x] (+)= sum over the k_parts partial sums, added in range order (deterministic). One thread per 4 columns.
template <int DT, bool ACCUMULATE>
__global__ __launch_bounds__(256) void lm_gemm_reduce_kernel(const float* __restrict__ partials, int64_t NX, int64_t NY,
                                                             int k_parts, uint16_t* __restrict__ out, int64_t out_stride) {
  using O = ElemOut<DT>;
  const int64_t quads_per_row = NX / 4;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= NY * quads_per_row) return;
  const int64_t y = idx / quads_per_row;
  const int64_t x = (idx % quads_per_row) * 4;
  f32x4 s = *reinterpret_cast<const f32x4*>(partials + y * NX + x);
  for (int p = 1; p < k_parts; ++p) {
    const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(partials + ((int64_t)p * NY + y) * NX + x));
    s += v;
  }
  uint2* dst = reinterpret_cast<uint2*>(out + y * out_stride + x);
  if constexpr (ACCUMULATE) {
    const uint2 old = *dst;
    float o[4];
    lm_unpack2<DT>(old.x, o);
    lm_unpack2<DT>(old.y, o + 2);
    s.x += o[0];
    s.y += o[1];
    s.z += o[2];
    s.w += o[3];
  }
  uint2 pk;
  pk.x = O::pack2(s.x, s.y);
  pk.y = O::pack2(s.z, s.w);
  *dst = pk;
}

// grid.x = ceil(T / 4), block = 256: wavefront w of a workgroup finishes token blockIdx.x * 4 + w.
template <int DT>
__global__ __launch_bounds__(256) void lmhead_finish_kernel(
    const char* __restrict__ W, const char* __restrict__ H, int64_t V, int64_t T, int64_t K, int64_t w_stride,
    int64_t h_stride, const int64_t* __restrict__ labels, const float* __restrict__ temperature, int n_runs,
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
  // The token's n_runs * 4 states (lmhead_partial_kernel: one per run of vocabulary tiles and wavefront quarter), in an
  // order that the vocabulary alone fixes: lane l takes states l, l + 64, ...; all are brought to the common maximum,
  // summed per lane in that order and then over the lanes.
  const int64_t n_states = static_cast<int64_t>(n_runs) * 4;
  const float* mine = partials + tok * n_states * 3;
  float M = neg_inf();
  for (int64_t i = lane; i < n_states; i += 64) M = __builtin_fmaxf(M, mine[i * 3]);
  M = wave_max(M);
  Part w;
  w.m = M;
  w.s = 0.f;
  w.t = 0.f;
  w.q = 0.f;
  for (int64_t i = lane; i < n_states; i += 64) {
    Part p;
    p.m = mine[i * 3];
    p.s = mine[i * 3 + 1];
    p.t = mine[i * 3 + 2];
    p.q = 0.f;
    rescale(p, M);
    w.s += p.s;
    w.t += p.t;
  }
  w.s = wave_sum(w.s);
  w.t = wave_sum(w.t);
  if (lane == 0) {
    const Scale<false> sc = make_scale<false>(temperature, tok);
    finalize_row<false, false>(w, xl, label_ok, sc, tok, out_logprob, out_entropy, nullptr, out_lse, err_flag);
  }
}

}  // namespace vrl
