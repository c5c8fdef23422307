// Layout shared by the producers and the consumer of the coarse-sorted scatter (csr_bin_scatter.hip,
// jitconn_ops.hip): products are appended to bins keyed by (producer, output window) and a second
// kernel adds each window's bins in a float64 window in LDS.
#pragma once

#include <cstdint>

namespace bpl {

constexpr uint32_t kBinWinShift = 14;  // output window = 16,384 elements (128 KB of float64)
constexpr uint32_t kBinWinCols = 1u << kBinWinShift;
constexpr uint32_t kBinMaxWindows = 128;  // 7-bit window ids

template <typename F>
struct BinPair {
  uint32_t rel;  // position within the window
  F val;
};

}  // namespace bpl
