// Workgroup shapes of the row kernels, shared by the launchers of the C ABI and by the bench-side memory probes (which
// read and copy with exactly these shapes).
#pragma once

#include "vrl.h"

namespace {

// Workgroup shape of the row kernel (wavefronts per row, 128-bit loads per lane
// and batch), chosen by measurement on MI355X at 8192 x 151936 and 32768 x 152064.
// Every shape from 1 to 16 wavefronts and 2 to 8 loads lands within 3 % of the
// others (6.7 to 7.05 TB/s, a plain read of the same rows reaches 7.05); these
// were on top at both sizes.
template <int DT>
struct RowShape;
template <>
struct RowShape<VRL_F32> {
  static constexpr int kWaves = 4, kUnroll = 4;
};
template <>
struct RowShape<VRL_BF16> {
  static constexpr int kWaves = 8, kUnroll = 2;
};
template <>
struct RowShape<VRL_F16> {
  static constexpr int kWaves = 8, kUnroll = 2;
};
// Shape of a workgroup that reduces one slice of a row (split path).
constexpr int kSplitWaves = 4;
constexpr int kSplitUnroll = 2;
constexpr int kMaxSplits = 64;
// Shape of the backward workgroup (one per row): wavefronts, 128-bit loads/stores per lane and batch.
// (measured 5.2-5.3 TB/s of read+write for every shape from 4 to 16 wavefronts, the same as a plain
// non-temporal copy of the same buffers)
constexpr int kBackwardWaves = 8;
constexpr int kBackwardUnroll = 2;

}  // namespace
