// Layout shared by the producers and the consumer of the coarse-sorted scatter (csr_bin_scatter.hip,
// jitconn_ops.hip): products are appended to bins keyed by (producer, output window) and a second
// kernel adds each window's bins in a float64 window in LDS.
#pragma once

#include <cstdint>

namespace bpl {

constexpr uint32_t kBinLdsShift = 14;     // accumulators a consumer holds in LDS: 16,384 (128 KB of float64)
constexpr uint32_t kBinMaxShift = 17;     // largest output window; one above 2^14 is added in slices of 2^14,
                                          // each slice reading the window's pairs again
constexpr uint32_t kBinMaxWindows = 128;  // 7-bit window ids

// log2 of the output window for n_out outputs: about 64 windows (many LDS counters for the
// producers to spread over, enough consumer workgroups) of at most 16,384 elements; wider windows
// only where the output (above two million elements) would need more than 128 of those.
inline uint32_t bin_window_shift(uint32_t n_out) {
  uint32_t shift = 8;
  while (shift < kBinLdsShift && (n_out >> shift) > 64u) ++shift;
  while (shift < kBinMaxShift && (n_out >> shift) >= kBinMaxWindows) ++shift;
  return shift;
}
inline uint32_t bin_lds_shift(uint32_t shift) { return shift < kBinLdsShift ? shift : kBinLdsShift; }

template <typename F>
struct BinPair {
  uint32_t rel;  // position within the window
  F val;
};

}  // namespace bpl
