// Stable least-significant-digit radix sort of (key, position) pairs for one batch of sparse ids.
// Replaces cub::DeviceRadixSort::SortPairs at csrc/core/preprocess.cu:105-109 of the reference.
#pragma once
#include "common.h"

namespace hctr {

constexpr int kSortBlock = 256;                 // threads per block (4 waves)
#ifndef HCTR_SORT_ITEMS
#define HCTR_SORT_ITEMS 16
#endif
constexpr int kSortItems = HCTR_SORT_ITEMS;     // keys per thread
constexpr int kSortTile = kSortBlock * kSortItems;
constexpr int kSortMaxDigitBits = 10;           // up to 1024 bins: 4 wave-private rows of 4 KiB in LDS

struct SortScratch {
  uint32_t *ghist = nullptr;   // [bins][blocks] per-block digit counts, scanned in place per bin
  uint32_t *bintot = nullptr;  // [bins] totals per digit value
  size_t blocks_cap = 0;
};

inline size_t sort_blocks(size_t n) { return (n + kSortTile - 1) / kSortTile; }
// a sort of at most this many tiles launches no scan kernel: every block of the scatter sums the raw per-block counts
// of its bins itself (the sum over so few blocks costs less than a launch)
constexpr uint32_t kSmallSortBlocks = 16;
// tiles of the scan / unique kernels of the preprocess (256 threads x 8 items), whatever the sort tile is
inline size_t scan_blocks(size_t n) { return (n + 2047) / 2048; }

// digit width of the first pass for a key of `bits` bits (the passes split the bits evenly)
inline int sort_first_digit_bits(int bits) {
  if (bits < 1) bits = 1;
  const int passes = (bits + kSortMaxDigitBits - 1) / kSortMaxDigitBits;
  return (bits + passes - 1) / passes;
}

// Sorts n pairs by the low `bits` bits of the key.  The value of element i is its position i (never
// materialised as an input).  keys_in is left untouched; tmp_k0/tmp_k1 and tmp_v0/tmp_v1 are ping-pong
// buffers of n elements; the sorted keys end in *keys_sorted (one of tmp_k0/tmp_k1) and the sorted
// positions in vals_out.  n == 0 is a no-op.  first_hist_done: scratch.ghist already holds the per-block counts of
// the first pass' digit (sort_first_digit_bits(bits) low bits, tiles of kSortTile keys), written by the kernel
// that made the keys.  long_runs: most keys are expected to repeat over long stretches of the input (the digit counts
// then add once per wave where a wave's keys agree).
template <typename K>
void radix_sort_positions(hipStream_t stream, const K *keys_in, uint32_t n, int bits, K *tmp_k0, K *tmp_k1,
                          uint32_t *tmp_v0, uint32_t *tmp_v1, uint32_t *vals_out, const SortScratch &scratch,
                          const K **keys_sorted, bool first_hist_done = false, bool long_runs = false);

extern template void radix_sort_positions<uint32_t>(hipStream_t, const uint32_t *, uint32_t, int, uint32_t *,
                                                    uint32_t *, uint32_t *, uint32_t *, uint32_t *,
                                                    const SortScratch &, const uint32_t **, bool, bool);
extern template void radix_sort_positions<uint64_t>(hipStream_t, const uint64_t *, uint32_t, int, uint64_t *,
                                                    uint64_t *, uint32_t *, uint32_t *, uint32_t *,
                                                    const SortScratch &, const uint64_t **, bool, bool);

} // namespace hctr
