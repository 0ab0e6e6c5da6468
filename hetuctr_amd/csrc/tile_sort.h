// Stable LSD radix sort of one batch's (sort key, position) pairs in passes + 1 launches ("tile-sorted" passes), for
// batches of up to kTileSortMaxTiles sort tiles.  Same result as radix_sort_positions (radix_sort.h), which replaces
// cub::DeviceRadixSort::SortPairs at csrc/core/preprocess.cu:105-109 of the reference; fewer, fatter launches.
//
// Between two passes the pairs are kept "tile-sorted": cut into tiles of the sort's tile size in the order the earlier
// passes established, every tile sorted (stably) by the next digit, with one row of a table per tile that says where
// every digit value starts inside the tile.  A pass is then ONE launch: block o produces the o-th tile of the order by
// that digit -- it reads the table, works out which pieces of which tiles its positions come from (pieces are
// contiguous in their tiles), fetches them, and sorts what it holds by the following digit for the next pass.  Counting
// a digit, scanning the counts and moving the pairs -- three dependent launches per pass in radix_sort.hip -- happen in
// the launch that has the data in its hands; no global atomics, no block waits for another.
//   launch 0            ids -> sort keys (make_keys' job), tiles sorted by digit 0
//   launch j, 0<j<P     tiles of the order by digits 0..j-1, sorted by digit j
//   launch P            the sorted keys and positions, and per wave-sized chunk of sorted positions what the unique pass
//                       needs to count unique keys before a position without a counting launch of its own
#pragma once
#include "kernels.h"
#include "radix_sort.h"

namespace hctr {

// Tile shape of these passes: keys per thread such that a batch makes at most kTileSortMaxTiles tiles (one block per
// tile and launch; 256 compute units) and as many of them as the shapes allow: the passes are latency, and the rounds
// a block spends ranking its keys are the longest piece of it.  Shapes: 2, 4, 8, 13 or 16 keys per thread.
#ifndef HCTR_TILE_SORT_MAX_TILES
#define HCTR_TILE_SORT_MAX_TILES 256
#endif
constexpr uint32_t kTileSortMaxTiles = HCTR_TILE_SORT_MAX_TILES;
constexpr int kTileItemsMax = 16;
constexpr inline int tile_items(size_t n) {
  const size_t per_thread = (n + (size_t)kTileSortMaxTiles * kSortBlock - 1) / ((size_t)kTileSortMaxTiles * kSortBlock);
#ifdef HCTR_TILE_NO_13
  return per_thread <= 2 ? 2 : per_thread <= 4 ? 4 : per_thread <= 8 ? 8 : 16;
#else
  return per_thread <= 2 ? 2 : per_thread <= 4 ? 4 : per_thread <= 8 ? 8 : per_thread <= 13 ? 13 : 16;
#endif
}
constexpr inline size_t tile_keys(size_t n) { return (size_t)kSortBlock * tile_items(n); }
constexpr inline size_t tile_count(size_t n) { return (n + tile_keys(n) - 1) / tile_keys(n); }
// The passes are used up to kTileSortMaxKeys keys.  Measured on an MI355X (whole training step, 26-bit keys, the sort
// beside the gradient push of the step before): they take 8-13 us off a step of 27 k to 430 k keys and 5-10 us off one
// of 0.85-1.3 M keys; at 1.7 M keys the step is 6 us longer than with the three-launch passes of radix_sort.h (the
// launches are fewer, but a block ranks its keys five times instead of three, and that arithmetic is what the push
// kernel beside it loses).
#ifndef HCTR_TILE_SORT_MAX_KEYS
#define HCTR_TILE_SORT_MAX_KEYS (3u << 19)
#endif
constexpr size_t kTileSortMaxKeys = HCTR_TILE_SORT_MAX_KEYS;
constexpr inline bool tile_sort_possible(size_t n) { return n != 0 && tile_count(n) <= kTileSortMaxTiles; }
constexpr inline bool tile_sort_fits(size_t n) { return n <= kTileSortMaxKeys && tile_sort_possible(n); }

// Per chunk of sorted positions (one wave's share of a tile: tile_items(n) * 64 positions): how many positions of the
// chunk other than its first hold another key than the position before, and the chunk's first and last key.
struct HeadChunks {
  uint32_t *inner = nullptr;   // [chunks]
  void *first = nullptr;       // [chunks] sort keys (K)
  void *last = nullptr;        // [chunks]
  uint32_t chunk = 0;          // positions per chunk
};
// storage for the head counts of an n-key batch in one allocation of head_chunk_words(n) words (inner, then first, then
// last; sized for the smallest chunk any path uses, 128 positions, and 64-bit keys)
constexpr inline size_t head_chunk_words(size_t n) { return ((n + 127) / 128) * 5 + 8; }
inline HeadChunks head_chunks_in(uint32_t *words, size_t n, bool wide, uint32_t chunk) {
  HeadChunks h;
  const size_t c = (n + chunk - 1) / chunk;
  h.inner = words;
  unsigned char *p = (unsigned char *)(words + (c + 1) / 2 * 2); // 8-byte aligned behind the counts
  h.first = p;
  h.last = p + c * (wide ? 8 : 4);
  h.chunk = chunk;
  return h;
}

// Words of table scratch the passes of n keys need: two tables (one read, one written by a launch) of two-byte entries,
// table[digit value][tile] = place of the first pair with that digit value in the tile, columns padded to 8 tiles.
constexpr inline size_t tile_table_pitch(size_t n) { return (tile_count(n) + 7) / 8 * 8; }
constexpr inline size_t tile_sort_table_words(size_t n) { return tile_table_pitch(n) * (size_t)kSortMaxBins; }

struct TileSortBuffers {
  void *keys[2];        // n sort keys each (ping-pong)
  uint32_t *vals[2];    // n positions each
  uint32_t *tables;     // tile_sort_table_words(n)
};

// Launch 0: reads the caller's ids (and nothing reads them afterwards), checks their range (bit 0 of *err), resets the
// batch's run counters (nlong, optional), writes the tiles sorted by the first digit into buffers 0.
// made_keys (optional): the batch's sort keys in batch order, already made and checked by make_keys; the launch then
// starts from them and looks at neither ids, err nor nlong.
// ids32: `ids` points to 32-bit ids (see launch_make_keys).  keys_out (optional, with ids): receives the sort keys in
// batch order as well.
void launch_tile_sort_keys(hipStream_t s, const TableView &t, const KeyLayout &kl, const index_t *ids,
                           const void *made_keys, uint32_t n, const TileSortBuffers &b, uint32_t *err, uint32_t *nlong,
                           bool ids32 = false, void *keys_out = nullptr);
// Launches [from, to) of the 1..P that follow (P = passes of kl.total_bits), for callers that enqueue them in pieces.
// The last one writes the sorted positions to sorted_arg, the sorted keys to *sorted_keys (one of b.keys) and `heads`.
// Returns P.
int launch_tile_sort_passes(hipStream_t s, const KeyLayout &kl, uint32_t n, const TileSortBuffers &b,
                            uint32_t *sorted_arg, const HeadChunks &heads, const void **sorted_keys, int from = 1,
                            int to = 1 << 30);
} // namespace hctr
