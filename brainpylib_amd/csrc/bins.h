// Layout shared by the producers and the consumer of the coarse-sorted scatter (csr_bin_scatter.hip,
// jitconn_ops.hip): products are appended to bins keyed by (producer, output window) and a second
// kernel adds each window's bins in a float64 window in LDS.
#pragma once

#include <cstdint>

namespace bpl {

constexpr uint32_t kBinMaxShift = 14;     // largest output window: 16,384 elements (128 KB of float64)
constexpr uint32_t kBinMaxWindows = 128;  // 7-bit window ids

// log2 of the output window for n_out outputs: about 64 windows (many LDS counters for the
// producers to spread over, enough consumer workgroups), at most 16,384 elements each.
inline uint32_t bin_window_shift(uint32_t n_out) {
  uint32_t shift = 8;
  while (shift < kBinMaxShift && (n_out >> shift) > 64u) ++shift;
  return shift;
}

template <typename F>
struct BinPair {
  uint32_t rel;  // position within the window
  F val;
};

}  // namespace bpl
