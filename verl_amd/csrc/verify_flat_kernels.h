// SPEC-RL draft verification as two flat passes over the tokens, for batches whose sequences differ widely in length.
//
// One workgroup per sequence (verify_kernels.h) leaves the longest sequence's bytes to a single CU: at 512 packed
// sequences of 32 ... 16384 tokens the CUs that hold the long ones move 5 x the average and the launch takes as long
// as they do. Here every workgroup owns a tile of kTile consecutive tokens of the arrays instead, whatever sequences
// they belong to, and what a sequence needs from its other tiles travels as one bit per token:
//
//   pass 1 (verify_tokens_kernel, grid = tiles): per token d = logp_new - logp_old, tau = log_u + offset, accept; per
//     64 tokens four ballot words in the workspace (S: a sequence starts here, R: valid and rejected, V: valid,
//     N: near the threshold); per tile a 3-bit summary (below).
//   pass 2 (verify_finish_kernel, grid = tiles + sequences / 4): a tile's workgroup turns S, R, V into KEEP bits with
//     word-parallel segmented fills (a token is kept iff no rejection lies between its sequence's start and itself and a
//     valid token lies between itself and its sequence's end), with the carries across its two borders taken from the
//     neighbouring tiles' summaries, and writes the truncated draft; one wavefront per sequence reads the sequence's R,
//     V, N words and writes first_reject, prefix_len and near_count.
//
// Every per-token byte is read or written once, by a workgroup chosen by the token's index alone; the words are 0.5
// bytes per token. Integer results only depend on the bits, so they equal verify_sequence's.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "verify_kernels.h"

namespace vrl {

constexpr int kTile = 1024;             // tokens per workgroup
constexpr int kTileWords = kTile / 64;  // ballot words per tile and kind
constexpr int kFlatThreads = 256;
constexpr int kDirectScanMax = 4096;    // packed batches of up to this many sequences: tiles scan cu_seqlens instead of searching it

// Tile summary bits: what the neighbouring tiles need to know about this one.
constexpr uint32_t kSumStart = 1;   // some sequence starts inside the tile
constexpr uint32_t kSumRejOut = 2;  // a rejection is pending at the tile's last token: one lies at or behind the tile's
                                    // last sequence start (behind its first token when no sequence starts inside)
constexpr uint32_t kSumValHead = 4; // a valid token lies before the tile's first sequence start (anywhere when none)

// Workspace layout (bytes): four arrays of n_words 64-bit words (S, R, V, N), then n_tiles 32-bit summaries.
struct FlatWork {
  unsigned long long* S;
  unsigned long long* R;
  unsigned long long* V;
  unsigned long long* N;
  uint32_t* summary;
  int64_t n_tiles;
};

__host__ __device__ inline int64_t flat_words(int64_t n_tokens) { return ((n_tokens + kTile - 1) / kTile) * kTileWords; }
__host__ __device__ inline int64_t flat_tiles(int64_t n_tokens) { return (n_tokens + kTile - 1) / kTile; }
__host__ __device__ inline int64_t flat_workspace_bytes(int64_t n_tokens) {
  return flat_words(n_tokens) * 4 * 8 + flat_tiles(n_tokens) * 4;
}
__host__ __device__ inline FlatWork flat_work(void* workspace, int64_t n_tokens) {
  FlatWork w;
  const int64_t nw = flat_words(n_tokens);
  w.S = static_cast<unsigned long long*>(workspace);
  w.R = w.S + nw;
  w.V = w.R + nw;
  w.N = w.V + nw;
  w.summary = reinterpret_cast<uint32_t*>(w.N + nw);
  w.n_tiles = flat_tiles(n_tokens);
  return w;
}

// Sum over the workgroup of a per-wavefront value (every thread of a wavefront passes the same v); 256 threads.
__device__ __forceinline__ int block_sum_of_waves(int v, int* sm) {
  const int wave = threadIdx.x >> 6;
  __syncthreads();   // sm may still be read from the round before
  if ((threadIdx.x & 63) == 0) sm[wave] = v;
  __syncthreads();
  return sm[0] + sm[1] + sm[2] + sm[3];
}

// Packed layout: mark in sS (kTileWords words in LDS, zeroed) every token of tile [t0, t0 + kTile) at which a sequence
// starts, i.e. every cu_seqlens[b], b < B, inside the tile. The entries are found with a cooperative search (each round
// 256 samples of the remaining index range, monotone offsets assumed) followed by a walk over the entries behind it.
// Offsets that are not monotone make the search end somewhere else; every index stays in [0, B] and only positions
// inside the tile are marked, so nothing but the marks depends on them.
__device__ __forceinline__ void mark_starts_packed(const int64_t* __restrict__ cu, int64_t B, int64_t t0,
                                                   unsigned long long* sS, int* sm) {
  const int tid = threadIdx.x;
  // number of entries cu[0 .. B] that are <= t0, by rounds of 256 samples: lo = entries known to be <= t0
  int64_t lo = 0, hi = B + 1;   // the answer lies in [lo, hi]
  while (hi - lo > 0) {
    const int64_t span = hi - lo;
    const int64_t step = (span + kFlatThreads - 1) / kFlatThreads;
    const int64_t idx = lo + static_cast<int64_t>(tid) * step + (step - 1);   // last entry of this thread's stretch
    const bool in = idx < hi;
    const bool le = in && (cu[idx] <= t0);
    const int c = block_sum_of_waves(__builtin_popcountll(__ballot(le)), sm);   // stretches that lie entirely <= t0
    const int64_t nlo = lo + static_cast<int64_t>(c) * step;
    int64_t nhi = nlo + step - 1;   // the first stretch whose last entry is > t0 may still hold entries <= t0
    if (nhi > hi) nhi = hi;
    if (nlo >= hi) {
      lo = hi;
      break;
    }
    if (step == 1) {   // stretches are single entries: entry nlo is > t0
      lo = nlo;
      hi = nlo;
      break;
    }
    lo = nlo;
    hi = nhi;
  }
  // entries lo, lo + 1, ... are > t0 (or lo == B + 1): walk them until one leaves the tile
  const int64_t t1 = t0 + kTile;
  // a sequence that starts exactly at t0 is entry lo - 1 (== t0) or earlier equal ones
  if (tid == 0 && lo > 0 && lo - 1 < B && cu[lo - 1] == t0) atomicOr(&sS[0], 1ull);
  for (int64_t base = lo;; base += kFlatThreads) {
    const int64_t idx = base + tid;
    bool inside = false;
    if (idx < B) {   // entry B is the end of the last sequence, not a start
      const int64_t p = cu[idx];
      inside = p < t1;
      if (p > t0 && p < t1) {
        const int rel = static_cast<int>(p - t0);
        atomicOr(&sS[rel >> 6], 1ull << (rel & 63));
      }
    }
    // go on only while every entry of this round was still inside the tile
    const int c = block_sum_of_waves(__builtin_popcountll(__ballot(inside)), sm);
    if (c < kFlatThreads) break;
  }
}

// Padded layout: sequences start at multiples of T. Word `word` of the whole token range.
__device__ __forceinline__ unsigned long long starts_padded_word(int64_t word, int64_t T, int64_t n_tokens) {
  const int64_t g0 = word * 64;
  if (g0 >= n_tokens || T <= 0) return 0ull;
  const int64_t r = g0 % T;
  unsigned long long w = 0ull;
  for (int64_t p = (r == 0) ? 0 : T - r; p < 64 && g0 + p < n_tokens; p += T) w |= 1ull << p;
  return w;
}

// grid.x = tiles, block = 256: wavefront w of a tile owns its words 4w .. 4w+3, lane l token l of each.
__global__ __launch_bounds__(kFlatThreads) void verify_tokens_kernel(const VerifyArgs v, const FlatWork ws) {
  __shared__ unsigned long long sS[kTileWords], sR[kTileWords], sV[kTileWords];
  __shared__ int sm[4];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t tile = blockIdx.x;
  const int64_t t0 = tile * kTile;

  // the token loads first: nothing below depends on them until the ballots
  float ln[4], lo[4], lu[4];
  uint8_t mk[4];
  bool in[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t g = t0 + (wave * 4 + j) * 64 + lane;
    in[j] = g < v.n_tokens;
    ln[j] = lo[j] = lu[j] = 0.f;
    mk[j] = 0;
    if (in[j]) {
      ln[j] = v.logp_new[g];
      lo[j] = v.logp_old[g];
      lu[j] = v.log_u[g];
      mk[j] = (v.mask != nullptr) ? v.mask[g] : static_cast<uint8_t>(1);
    }
  }

  if (tid < kTileWords) sS[tid] = 0ull;
  __syncthreads();
  if (v.cu_seqlens != nullptr) {
    if (v.B <= kDirectScanMax) {
      // few sequences: every tile looks at every offset (independent loads, in flight together with the token loads,
      // from an array that stays in L2) instead of searching for its own
      const int64_t t1 = t0 + kTile;
#pragma unroll
      for (int k = 0; k < kDirectScanMax / kFlatThreads; ++k) {
        const int64_t idx = static_cast<int64_t>(k) * kFlatThreads + tid;
        if (idx < v.B) {
          const int64_t p = v.cu_seqlens[idx];
          if (p >= t0 && p < t1) {
            const int rel = static_cast<int>(p - t0);
            atomicOr(&sS[rel >> 6], 1ull << (rel & 63));
          }
        }
      }
    } else {
      mark_starts_packed(v.cu_seqlens, v.B, t0, sS, sm);
    }
  } else if (lane < 4) {
    const int w = wave * 4 + lane;
    sS[w] = starts_padded_word(tile * kTileWords + w, v.T, v.n_tokens);
  }

#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int w = wave * 4 + j;
    const float d = ln[j] - lo[j];
    const float tau = lu[j] + v.thresh_offset;
    const bool valid = in[j] && (mk[j] != 0);
    const bool ok = d >= tau;
    const bool close = valid && (__builtin_fabsf(d - tau) < v.near_eps);
    if (in[j]) v.accept[t0 + w * 64 + lane] = static_cast<uint8_t>(valid && ok);
    const unsigned long long rej = __ballot(valid && !ok);
    const unsigned long long val = __ballot(valid);
    const unsigned long long nr = __ballot(close);
    if (lane == 0) {
      const int64_t gw = tile * kTileWords + w;
      ws.R[gw] = rej;
      ws.V[gw] = val;
      ws.N[gw] = nr;
      sR[w] = rej;
      sV[w] = val;
    }
  }
  __syncthreads();   // sS, sR, sV complete
  if (wave == 0) {
    const bool has = lane < kTileWords;
    const unsigned long long S = has ? sS[lane] : 0ull;
    const unsigned long long R = has ? sR[lane] : 0ull;
    const unsigned long long V = has ? sV[lane] : 0ull;
    if (has) ws.S[tile * kTileWords + lane] = S;
    const unsigned long long smask = __ballot(S != 0ull);
    uint32_t sum = 0;
    if (smask != 0ull) {
      const int w_hi = 63 - __builtin_clzll(smask), w_lo = __builtin_ctzll(smask);
      // rejections at or behind the last start; valid tokens before the first start
      const int s_hi = S != 0ull ? 63 - __builtin_clzll(S) : 0, s_lo = S != 0ull ? __builtin_ctzll(S) : 0;
      bool r_after = lane > w_hi && R != 0ull;
      if (lane == w_hi) r_after = (R >> s_hi) != 0ull;
      bool v_before = lane < w_lo && V != 0ull;
      if (lane == w_lo) v_before = (V & ((1ull << s_lo) - 1ull)) != 0ull;
      sum = kSumStart | (__ballot(r_after) != 0ull ? kSumRejOut : 0u) | (__ballot(v_before) != 0ull ? kSumValHead : 0u);
    } else {
      sum = (__ballot(R != 0ull) != 0ull ? kSumRejOut : 0u) | (__ballot(V != 0ull) != 0ull ? kSumValHead : 0u);
    }
    if (lane == 0) ws.summary[tile] = sum;
  }
}

// Forward fill inside a word: bit i of the result is set iff some set bit j <= i of `gen` has no set bit of `stop` in
// (j, i]. (Kogge-Stone over 64 bits; a stop bit blocks what arrives from below, not what is generated on it.)
__device__ __forceinline__ unsigned long long fill_up(unsigned long long gen, unsigned long long stop) {
  unsigned long long pro = ~stop;
#pragma unroll
  for (int sh = 1; sh < 64; sh <<= 1) {
    gen |= pro & (gen << sh);
    pro &= pro << sh;
  }
  return gen;
}

// Backward fill: bit i is set iff some set bit j >= i of `gen` has no set bit of `stop` in (i, j]: token i and token
// i + 1 share a sequence iff no sequence starts at i + 1.
__device__ __forceinline__ unsigned long long fill_down(unsigned long long gen, unsigned long long stop) {
  unsigned long long pro = ~(stop >> 1);   // bit i: may receive from bit i + 1 (bit 63 receives nothing inside the word)
#pragma unroll
  for (int sh = 1; sh < 64; sh <<= 1) {
    gen |= pro & (gen >> sh);
    pro &= pro >> sh;
  }
  return gen;
}

// One wavefront: the carries a tile receives from its neighbours. rej_in: "a rejection is pending when the tile's first
// token is reached", settled by the nearest tile before it that has kSumRejOut (yes) or a sequence start (no);
// val_in: "a valid token of the same sequence follows the tile's last token", settled by the nearest tile behind it with
// kSumValHead (yes) or a sequence start (no). A tile that does not exist settles with no. 64 summaries per direction
// and round, both directions requested together.
__device__ __forceinline__ void tile_carries(const uint32_t* __restrict__ summary, int64_t n_tiles, int64_t tile,
                                             bool* rej_in, bool* val_in) {
  const int lane = threadIdx.x & 63;
  bool need_r = true, need_v = true;
  *rej_in = false;
  *val_in = false;
  for (int64_t off = 1; need_r || need_v; off += 64) {
    const int64_t tp = tile - (off + lane), tn = tile + (off + lane);
    const bool ep = tp >= 0, en = tn < n_tiles;
    const uint32_t sp = (need_r && ep) ? summary[tp] : 0u;
    const uint32_t sn = (need_v && en) ? summary[tn] : 0u;
    if (need_r) {
      const unsigned long long settles = __ballot(!ep || (sp & (kSumRejOut | kSumStart)) != 0u);
      if (settles != 0ull) {
        const uint32_t sf = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(sp), __builtin_ctzll(settles)));
        *rej_in = (sf & kSumRejOut) != 0u;
        need_r = false;
      }
    }
    if (need_v) {
      const unsigned long long settles = __ballot(!en || (sn & (kSumValHead | kSumStart)) != 0u);
      if (settles != 0ull) {
        const uint32_t sf = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(sn), __builtin_ctzll(settles)));
        *val_in = (sf & kSumValHead) != 0u;
        need_v = false;
      }
    }
  }
}

// The 64-bit value that lane `src` (wave-uniform) holds.
__device__ __forceinline__ unsigned long long readlane_u64(unsigned long long x, int src) {
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(x)), src));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(x >> 32)), src));
  return (static_cast<unsigned long long>(hi) << 32) | lo;
}

// One wavefront per sequence: first_reject, prefix_len, near_count from the sequence's R, V, N words.
__device__ __forceinline__ void finish_sequence(const VerifyArgs& v, const FlatWork& ws, int64_t b) {
  const int lane = threadIdx.x & 63;
  int64_t lo, hi;
  if (v.cu_seqlens != nullptr) {
    lo = v.cu_seqlens[b];
    hi = v.cu_seqlens[b + 1];
    const bool bad = (lo < 0) || (hi > v.n_tokens) || (hi < lo) || (b == 0 && lo != 0) || (b + 1 == v.B && hi != v.n_tokens);
    if (bad && lane == 0 && v.err_flag != nullptr) atomicOr(v.err_flag, kFlagSeqRange);
    lo = lo < 0 ? 0 : (lo > v.n_tokens ? v.n_tokens : lo);
    hi = hi < lo ? lo : (hi > v.n_tokens ? v.n_tokens : hi);
  } else {
    lo = b * v.T;
    hi = lo + v.T;
  }
  int first = kNoReject, last_valid = 0, near = 0, before = 0;   // wave-uniform; `before`: valid tokens ahead of `first`
  if (hi > lo) {
    const int64_t w0 = lo >> 6, w1 = (hi - 1) >> 6;
    for (int64_t wb = w0; wb <= w1; wb += 64) {
      const int64_t w = wb + lane;
      unsigned long long R = 0ull, V = 0ull, N = 0ull;
      if (w <= w1) {
        unsigned long long m = ~0ull;
        if (w == w0) m &= ~0ull << (lo & 63);
        if (w == w1) m &= ~0ull >> (63 - ((hi - 1) & 63));
        N = ws.N[w] & m;
        V = ws.V[w] & m;
        if (first == kNoReject) R = ws.R[w] & m;
      }
      near += __builtin_popcountll(N);
      const unsigned long long vb = __ballot(V != 0ull);
      if (vb != 0ull) {
        const int ll = 63 - __builtin_clzll(vb);
        const int hb = 63 - __builtin_clzll(readlane_u64(V, ll));
        last_valid = static_cast<int>((wb + ll) * 64 + hb + 1 - lo);
      }
      if (first == kNoReject) {
        const unsigned long long rb = __ballot(R != 0ull);
        if (rb != 0ull) {
          const int fl = __builtin_ctzll(rb);
          const int bit = __builtin_ctzll(readlane_u64(R, fl));
          first = static_cast<int>((wb + fl) * 64 + bit - lo);
          // valid tokens of this round that lie before it
          int c = 0;
          if (lane < fl) c = __builtin_popcountll(V);
          if (lane == fl) c = __builtin_popcountll(V & ((1ull << bit) - 1ull));
          before += c;
        } else {
          before += __builtin_popcountll(V);
        }
      }
    }
    near = wave_sum_int(near);
    before = wave_sum_int(before);
  }
  if (lane == 0) {
    // without a rejection the prefix ends behind the last valid token, and every valid token lies before that
    v.first_reject[b] = first == kNoReject ? last_valid : first;
    v.prefix_len[b] = before;
    v.near_count[b] = near;
  }
}

// grid.x = tiles (only when a truncated draft is asked for, else 0) + ceil(B / 4), block = 256.
__global__ __launch_bounds__(kFlatThreads) void verify_finish_kernel(const VerifyArgs v, const FlatWork ws,
                                                                     int64_t n_draft_tiles) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (static_cast<int64_t>(blockIdx.x) >= n_draft_tiles) {
    const int64_t b = (static_cast<int64_t>(blockIdx.x) - n_draft_tiles) * 4 + wave;
    if (b < v.B) finish_sequence(v, ws, b);
    return;   // this workgroup has no barrier
  }
  __shared__ unsigned long long sKeep[kTileWords], sVal[kTileWords];
  const int64_t tile = blockIdx.x;
  const int64_t t0 = tile * kTile;
  if (wave == 0) {
    const bool has = lane < kTileWords;
    const unsigned long long S = has ? ws.S[tile * kTileWords + lane] : 0ull;
    const unsigned long long R = has ? ws.R[tile * kTileWords + lane] : 0ull;
    const unsigned long long V = has ? ws.V[tile * kTileWords + lane] : 0ull;
    bool rej_in, val_in;
    tile_carries(ws.summary, ws.n_tiles, tile, &rej_in, &val_in);
    // inside each word
    unsigned long long A = fill_up(R, S);     // a rejection between the sequence's start (or the word's) and the token
    unsigned long long Bv = fill_down(V, S);  // a valid token between the token and the sequence's end (or the word's)
    // across the words of the tile: what enters word w from below (rejection pending) and from above (valid follows)
    const unsigned long long has_s = __ballot(S != 0ull);
    const unsigned long long a_out = __ballot((A >> 63) != 0ull);                  // pending at the word's last token
    const unsigned long long b_out = __ballot((Bv & 1ull) != 0ull && (S & 1ull) == 0ull);   // reaches the token before the word
    bool cin_a = rej_in;
    for (int w = 0; w < lane && w < kTileWords; ++w)
      cin_a = ((a_out >> w) & 1ull) != 0ull || (cin_a && ((has_s >> w) & 1ull) == 0ull);
    bool cin_b = val_in;
    for (int w = kTileWords - 1; w > lane; --w)
      cin_b = ((b_out >> w) & 1ull) != 0ull || (cin_b && ((has_s >> w) & 1ull) == 0ull);
    // a carry from below covers the tokens before the word's first start; one from above the tokens from its last start on
    const int s_hi = S != 0ull ? 63 - __builtin_clzll(S) : 0, s_lo = S != 0ull ? __builtin_ctzll(S) : 0;
    if (cin_a) A |= (S == 0ull) ? ~0ull : ((1ull << s_lo) - 1ull);
    if (cin_b) Bv |= (S == 0ull) ? ~0ull : (~0ull << s_hi);
    if (has) {
      sKeep[lane] = ~A & Bv;
      sVal[lane] = V;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int w = wave * 4 + j;
    const int64_t g = t0 + w * 64 + lane;
    if (g < v.n_tokens) {
      const bool keep = ((sKeep[w] >> lane) & 1ull) != 0ull;
      const bool valid = ((sVal[w] >> lane) & 1ull) != 0ull;
      v.out_ids[g] = keep ? v.draft_ids[g] : v.pad_id;
      v.out_mask[g] = static_cast<uint8_t>(keep && valid);
    }
  }
}

}  // namespace vrl
