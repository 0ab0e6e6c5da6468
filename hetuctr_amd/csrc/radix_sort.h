// Stable least-significant-digit radix sort of (key, position) pairs for one batch of sparse ids.
// Replaces cub::DeviceRadixSort::SortPairs at csrc/core/preprocess.cu:105-109 of the reference.
#pragma once
#include "common.h"

namespace hctr {

#ifndef HCTR_SORT_BLOCK
#define HCTR_SORT_BLOCK 512
#endif
constexpr int kSortBlock = HCTR_SORT_BLOCK;     // threads per block
constexpr int kSortMaxDigitBits = 10;           // up to 1024 bins
constexpr int kSortMaxBins = 1 << kSortMaxDigitBits;
// Keys per thread, hence keys per tile (one block sorts one tile per pass), chosen by the size of the input: a small
// input is cut into small tiles so that enough blocks share it (its passes are latency, not traffic); a large one into
// large tiles, because every tile costs a row of digit counts that is written, scanned and read again in every pass,
// and because fewer, longer-lived blocks take less from a kernel that runs beside the sort on another stream (at
// 1.7 M keys the sort alone is 4 us slower with 8192-key tiles than with 4096-key ones, the step beside it 5 us faster).
#ifndef HCTR_SORT_ITEMS_DEFAULT
#define HCTR_SORT_ITEMS_DEFAULT 8
#endif
#ifndef HCTR_SORT_ITEMS_LARGE
#define HCTR_SORT_ITEMS_LARGE 16
#endif
#ifndef HCTR_SORT_ITEMS_SMALL
#define HCTR_SORT_ITEMS_SMALL 2
#endif
constexpr int kSortItemsSmall = HCTR_SORT_ITEMS_SMALL, kSortItemsDefault = HCTR_SORT_ITEMS_DEFAULT, kSortItemsLarge = HCTR_SORT_ITEMS_LARGE;
constexpr size_t kSortSmallUpTo = (size_t)1 << 17, kSortLargeFrom = (size_t)1 << 20;
constexpr inline int sort_items(size_t n) {
  return n <= kSortSmallUpTo ? kSortItemsSmall : (n >= kSortLargeFrom ? kSortItemsLarge : kSortItemsDefault);
}
constexpr inline size_t sort_tile(size_t n) { return (size_t)kSortBlock * sort_items(n); }
constexpr inline size_t sort_tiles(size_t n) { return (n + sort_tile(n) - 1) / sort_tile(n); }
// words of scratch a sort of n keys needs: per tile and bin the count of the digit in the earlier tiles (of its piece of
// the scan), then the total of every bin (per piece).  Not monotonic in n (the tile grows with it): size the scratch for the n that is sorted.
// An input of many tiles has its count columns scanned in up to kScanMaxChunks pieces of at least kScanChunkRows rows,
// one block per piece and group of columns (a column of thousands of rows scanned by one block is a long serial
// walk); every piece leaves its column totals, which the scatter adds up.
#ifndef HCTR_SCAN_MAX_CHUNKS
#define HCTR_SCAN_MAX_CHUNKS 16
#endif
constexpr uint32_t kScanMaxChunks = HCTR_SCAN_MAX_CHUNKS, kScanChunkRows = 256;
constexpr inline uint32_t scan_chunks(size_t tiles) {
  const size_t c = tiles / kScanChunkRows;
  return c < 2 ? 1u : (c > kScanMaxChunks ? kScanMaxChunks : (uint32_t)c);
}
constexpr inline size_t sort_scratch_words(size_t n) { return (sort_tiles(n) + scan_chunks(sort_tiles(n))) * (size_t)kSortMaxBins; }
// the most words any input of up to n_max keys needs
inline size_t sort_scratch_words_upto(size_t n_max) {
  size_t w = sort_scratch_words(n_max);
  if (n_max > kSortSmallUpTo) w = w > sort_scratch_words(kSortSmallUpTo) ? w : sort_scratch_words(kSortSmallUpTo);
  if (n_max > kSortLargeFrom - 1) w = w > sort_scratch_words(kSortLargeFrom - 1) ? w : sort_scratch_words(kSortLargeFrom - 1);
  return w;
}
// expands CALL(ITEMS) for the tile shape of an input of n keys
#define HCTR_SORT_ITEMS_DISPATCH(n, CALL)                      \
  do {                                                         \
    switch (::hctr::sort_items(n)) {                           \
      case ::hctr::kSortItemsSmall: CALL(::hctr::kSortItemsSmall); break;     \
      case ::hctr::kSortItemsLarge: CALL(::hctr::kSortItemsLarge); break;     \
      default: CALL(::hctr::kSortItemsDefault); break;         \
    }                                                          \
  } while (0)

struct SortScratch {
  uint32_t *words = nullptr;   // sort_scratch_words(n) of them
  size_t n_cap = 0;            // the n they were sized for
};
// tiles of the scan / unique kernels of the preprocess (256 threads x 8 items), whatever the sort tile is
constexpr inline size_t scan_blocks(size_t n) { return (n + 2047) / 2048; }

// digit width of the first pass for a key of `bits` bits (the passes split the bits evenly)
inline int sort_first_digit_bits(int bits) {
  if (bits < 1) bits = 1;
  const int passes = (bits + kSortMaxDigitBits - 1) / kSortMaxDigitBits;
  return (bits + passes - 1) / passes;
}

// One key's digit into the block's LDS counters h[].  Called by every lane of the wave with consecutive keys in
// consecutive lanes; lanes inside the input (`in`) are a prefix of the wave.  A run of equal digits in consecutive
// lanes (what a partly sorted input and a hot key make of most waves) adds once, from its first lane, so that the
// LDS atomics of one instruction rarely meet on one word.
__device__ __forceinline__ void count_digit(uint32_t *h, uint32_t d, bool in) {
  const unsigned lane = lane_id();
  const uint32_t dp = __shfl_up(d, 1, kWave);
  const bool head = in && (lane == 0 || d != dp);
  const uint64_t act = __ballot(in);
  const uint64_t heads = __ballot(head);
  if (head) {
    const uint64_t above = lane == 63 ? 0ull : (heads >> (lane + 1));
    const uint32_t end = above ? lane + 1 + (uint32_t)__builtin_ctzll(above) : (uint32_t)__popcll(act);
    atomicAdd(&h[d], end - lane);
  }
}

// Sorts n pairs by the low `bits` bits of the key.  The value of element i is its position i (never
// materialised as an input).  keys_in is left untouched; tmp_k0/tmp_k1 and tmp_v0/tmp_v1 are ping-pong
// buffers of n elements; the sorted keys end in *keys_sorted (one of tmp_k0/tmp_k1) and the sorted
// positions in vals_out.  n == 0 is a no-op.  Three launches per pass of up to kSortMaxDigitBits bits.
// first_counts_done: scratch.words already holds the per-tile counts of the first pass' digit
// (sort_first_digit_bits(bits) low bits, rows of 1 << that many words, tiles of sort_tile(n) keys), written by the
// kernel that made the keys (see count_digit); its tiles are those of sort_tile(n).
// step_from / step_to: only the launches [step_from, step_to) of the sort are enqueued by this call, launch 3 * p + k
// being the count (k = 0), the column scan (1) or the scatter (2) of pass p; a caller that enqueues the sort in
// pieces passes the same other arguments every time.
template <typename K>
void radix_sort_positions(hipStream_t stream, const K *keys_in, uint32_t n, int bits, K *tmp_k0, K *tmp_k1,
                          uint32_t *tmp_v0, uint32_t *tmp_v1, uint32_t *vals_out, const SortScratch &scratch,
                          const K **keys_sorted, bool first_counts_done = false, int step_from = 0,
                          int step_to = 1 << 30);

extern template void radix_sort_positions<uint32_t>(hipStream_t, const uint32_t *, uint32_t, int, uint32_t *,
                                                    uint32_t *, uint32_t *, uint32_t *, uint32_t *,
                                                    const SortScratch &, const uint32_t **, bool, int, int);
extern template void radix_sort_positions<uint64_t>(hipStream_t, const uint64_t *, uint32_t, int, uint64_t *,
                                                    uint64_t *, uint32_t *, uint32_t *, uint32_t *,
                                                    const SortScratch &, const uint64_t **, bool, int, int);

} // namespace hctr
