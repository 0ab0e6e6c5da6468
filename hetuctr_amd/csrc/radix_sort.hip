// Stable LSD radix sort for gfx950, 64-lane wavefronts.
//
// One pass = three launches (two for a small input, see kSelfScanTiles), nothing waits on another block inside a kernel and no global atomics are used
// (device-scope atomics are two orders of magnitude slower than plain stores on this part):
//   digit_histogram   per-tile digit counts -> counts[tile][bin], rows written whole
//   scan_tiles        per bin: exclusive scan of its column over the tiles + the bin's total
//   scatter           one block per tile: global base of every bin, stable rank of every key inside the tile
//                     (wave-level match by ballots, wave-private LDS counters), the tile sorted by digit in LDS,
//                     then stores that are contiguous per bin
// Stability: a block's tile is split into 8 contiguous sub-tiles, one per wave; a wave walks its sub-tile 64 keys
// at a time in ascending position; inside such a group the rank among equal digits is the lane order.
// Wave-private counters make the result independent of wave scheduling.
#include "radix_sort.h"

namespace hctr {
namespace {

constexpr int kWaves = kSortBlock / kWave;
constexpr uint32_t kXcds = 8;              // accelerator dies of the device, each with its own L2
// A tile of ITEMS * kSortBlock keys: wave w takes the w-th run of ITEMS * 64 consecutive keys, 64 keys per round.
static_assert(kSortMaxBins <= 2 * kSortBlock, "a thread owns at most two bins");
static_assert(kSortBlock <= 1024 && kSortBlock % kWave == 0, "block shape");

// Digit counts of one tile: row `tile` of counts[tile][bin].  A run of equal digits in consecutive lanes (what a
// partly sorted input and a hot key make of most waves) adds once, from its first lane, so that the LDS atomics
// of one instruction rarely meet on one word.
template <typename K, int ITEMS>
__global__ __launch_bounds__(kSortBlock) void digit_histogram(const K *__restrict__ keys, uint32_t n, int shift,
                                                              int dbits, uint32_t *__restrict__ counts) {
  __shared__ uint32_t h[kSortMaxBins];
  const uint32_t nb = 1u << dbits, mask = nb - 1;
  constexpr uint32_t kTile = ITEMS * kSortBlock;
  K key[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t idx = blockIdx.x * kTile + k * kSortBlock + threadIdx.x;
    key[k] = idx < n ? keys[idx] : (K)0;
  }
  for (uint32_t i = threadIdx.x; i < nb; i += kSortBlock) h[i] = 0;
  __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t idx = blockIdx.x * kTile + k * kSortBlock + threadIdx.x;
    count_digit(h, (uint32_t)(key[k] >> shift) & mask, idx < n);
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < nb; i += kSortBlock) counts[(size_t)blockIdx.x * nb + i] = h[i];
}

// counts[tile][bin] -> in place, the count of the bin in the earlier tiles of the block's piece of the rows;
// bin_total[piece][bin].  A block scans kScanCols neighbouring bins: thread (part, col) adds up its part of the tiles for one bin.  Up to kScanKeep rows per thread
// stay in registers between the sum and the rewrite (one trip to memory); longer parts are read twice.
#ifndef HCTR_SCAN_COLS
#define HCTR_SCAN_COLS 16
#endif
#ifndef HCTR_SELF_SCAN_TILES
#define HCTR_SELF_SCAN_TILES 64
#endif
constexpr int kScanBlock = 512, kScanCols = HCTR_SCAN_COLS, kScanParts = kScanBlock / kScanCols, kScanKeep = 16;
__global__ __launch_bounds__(kScanBlock) void scan_tiles(uint32_t *__restrict__ counts, uint32_t tiles, uint32_t nb,
                                                         uint32_t *__restrict__ bin_total) {
  __shared__ uint32_t part_sum[kScanParts][kScanCols];
  const uint32_t c = threadIdx.x % kScanCols, col = blockIdx.x * kScanCols + c, part = threadIdx.x / kScanCols;
  // blockIdx.y: the piece of the rows this block scans (one piece: the whole column)
  const uint32_t rows_per = (tiles + gridDim.y - 1) / gridDim.y;
  const uint32_t clo = min(blockIdx.y * rows_per, tiles), chi = min(clo + rows_per, tiles);
  const uint32_t per = (chi - clo + kScanParts - 1) / kScanParts;
  const uint32_t lo = min(clo + part * per, chi), hi = min(lo + per, chi);
  const bool ok = col < nb;
  uint32_t first[kScanKeep];
#pragma unroll
  for (int u = 0; u < kScanKeep; u++) first[u] = (ok && lo + u < hi) ? counts[(size_t)(lo + u) * nb + col] : 0u;
  uint32_t s = 0;
#pragma unroll
  for (int u = 0; u < kScanKeep; u++) s += first[u];
  for (uint32_t t0 = lo + kScanKeep; t0 < hi; t0 += kScanKeep) {
    uint32_t v[kScanKeep];
#pragma unroll
    for (int u = 0; u < kScanKeep; u++) v[u] = (ok && t0 + u < hi) ? counts[(size_t)(t0 + u) * nb + col] : 0u;
#pragma unroll
    for (int u = 0; u < kScanKeep; u++) s += v[u];
  }
  part_sum[part][c] = s;
  __syncthreads();
  uint32_t run = 0;
  for (uint32_t q = 0; q < part; q++) run += part_sum[q][c];
  if (part == kScanParts - 1 && ok) bin_total[blockIdx.y * nb + col] = run + s; // the piece's total of the column
#pragma unroll
  for (int u = 0; u < kScanKeep; u++) {
    if (ok && lo + u < hi) counts[(size_t)(lo + u) * nb + col] = run;
    run += first[u];
  }
  for (uint32_t t0 = lo + kScanKeep; t0 < hi; t0 += kScanKeep) {
    uint32_t v[kScanKeep];
#pragma unroll
    for (int u = 0; u < kScanKeep; u++) v[u] = (ok && t0 + u < hi) ? counts[(size_t)(t0 + u) * nb + col] : 0u;
#pragma unroll
    for (int u = 0; u < kScanKeep; u++) {
      if (ok && t0 + u < hi) counts[(size_t)(t0 + u) * nb + col] = run;
      run += v[u];
    }
  }
}

// An input of at most this many tiles is sorted without the scan launches: every scatter block adds up the columns of
// the raw counts itself (a few rows from L2 cost less than a launch on a chain of dependent kernels).
constexpr uint32_t kSelfScanTiles = HCTR_SELF_SCAN_TILES;
constexpr int kSelfScanAhead = 32;         // rows of counts requested together

// DBITS: the digit width if known at compile time (the match loop is then straight-line code), else 0
// kMode 0: tile_prefix / bin_total are the scanned counts and the totals of one piece
//       1: tile_prefix holds the raw counts of digit_histogram (no scan launch), bin_total is not read
//       2: the scan ran in `pieces` pieces: tile_prefix counts inside the tile's piece, bin_total[piece][bin] adds up
template <typename K, bool kFirst, int ITEMS, int DBITS, int kMode>
__global__ __launch_bounds__(kSortBlock) void scatter(const K *__restrict__ keys_in, const uint32_t *__restrict__ vals_in,
                                                      K *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
                                                      uint32_t n, int shift, int dbits, uint32_t tiles,
                                                      const uint32_t *__restrict__ tile_prefix,
                                                      const uint32_t *__restrict__ bin_total, uint32_t pieces) {
#ifndef HCTR_SORT_NO_XCD
  // Workgroups go to the 8 XCDs of the device in turn, and each XCD has an L2 of its own.  XCD x takes the x-th
  // eighth of the tiles: neighbouring tiles write neighbouring pieces of every bin, so the pieces meet in one L2 and
  // leave it as whole lines.
  const uint32_t tiles_per_xcd = gridDim.x / kXcds;
  const uint32_t tile = (blockIdx.x % kXcds) * tiles_per_xcd + blockIdx.x / kXcds;
  if (tile >= tiles) return;
#else
  const uint32_t tile = blockIdx.x;
#endif
  constexpr int kRounds = ITEMS;                   // 64-key groups per wave
  constexpr int kSub = ITEMS * kWave;              // keys per wave
  constexpr uint32_t kSortTile = ITEMS * kSortBlock;
  // one LDS area, used twice: first the wave-private digit counters, then the tile sorted by digit
  constexpr int kCntWords = kWaves * kSortMaxBins;
  constexpr int kTileWords = (int)kSortTile * (int)(sizeof(K) / 4 + 1);
  __shared__ __align__(8) uint32_t area[kCntWords > kTileWords ? kCntWords : kTileWords];
  __shared__ uint32_t base[kSortMaxBins];      // global position of the bin's first key of this tile
  __shared__ uint32_t bin_start[kSortMaxBins]; // position of the bin inside the tile sorted by digit
  __shared__ uint32_t sm[kWaves + 1];
  uint32_t(*cnt)[kSortMaxBins] = (uint32_t(*)[kSortMaxBins])area;
  K *skey = (K *)area;
  uint32_t *sval = area + kSortTile * (sizeof(K) / 4);
  const uint32_t nb = 1u << dbits, mask = nb - 1;
  const int w = threadIdx.x / kWave;
  const unsigned lane = lane_id();
  // consecutive bins per thread in the scans over the bins
  const uint32_t per = nb > (uint32_t)kSortBlock ? nb / kSortBlock : 1u;
  const uint32_t blo = min(threadIdx.x * per, nb), bhi = min(blo + per, nb);

  // the keys of the tile: requested first, used after the bases are known
  K key[kRounds];
  uint32_t val[kRounds];
  const uint32_t wbase = tile * kSortTile + w * kSub;
#pragma unroll
  for (int r = 0; r < kRounds; r++) {
    const uint32_t idx = wbase + r * kWave + lane;
    const bool valid = idx < n;
    key[r] = valid ? load_once(&keys_in[idx]) : (K)0; // a pass reads its input once
    val[r] = kFirst ? idx : (valid ? load_once(&vals_in[idx]) : 0u);
  }

  // global position of each bin's first key of this tile: totals of the lower bins + this bin's count in the
  // earlier tiles
  {
    uint32_t all[2] = {0, 0}, mine[2] = {0, 0};
    if (kMode != 0) {
      // a table of rows to add up per bin: all of them for the bin's total, those before `rows_mine` for this tile
      const uint32_t *rows = kMode == 1 ? tile_prefix : bin_total;
      const uint32_t n_rows = kMode == 1 ? tiles : pieces;
      const uint32_t rows_mine = kMode == 1 ? tile : tile / ((tiles + pieces - 1) / pieces);
      for (int q = 0; q < 2; q++) {
        if (blo + q < bhi) {
          const uint32_t *col = rows + blo + q;
          for (uint32_t t0 = 0; t0 < n_rows; t0 += kSelfScanAhead) {
            uint32_t v[kSelfScanAhead];
#pragma unroll
            for (int u = 0; u < kSelfScanAhead; u++) v[u] = t0 + u < n_rows ? col[(size_t)(t0 + u) * nb] : 0u;
#pragma unroll
            for (int u = 0; u < kSelfScanAhead; u++) {
              all[q] += v[u];
              mine[q] += t0 + u < rows_mine ? v[u] : 0u;
            }
          }
          if (kMode == 2) mine[q] += tile_prefix[(size_t)tile * nb + blo + q];
        }
      }
    } else {
#pragma unroll
      for (int q = 0; q < 2; q++) {
        if (blo + q < bhi) {
          all[q] = bin_total[blo + q];
          mine[q] = tile_prefix[(size_t)tile * nb + blo + q];
        }
      }
    }
    uint32_t total;
    uint32_t off = block_exclusive_scan<kSortBlock>(all[0] + all[1], sm, total);
#pragma unroll
    for (int q = 0; q < 2; q++) {
      if (blo + q < bhi) {
        base[blo + q] = off + mine[q];
        off += all[q];
      }
    }
  }
  for (uint32_t i = threadIdx.x; i < kWaves * nb; i += kSortBlock) cnt[i / nb][i % nb] = 0;
  __syncthreads();

  // stable rank of every key among the keys of its wave with the same digit
  uint32_t dig[kRounds];
  uint32_t rnk[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; r++) {
    const uint32_t idx = wbase + r * kWave + lane;
    const bool valid = idx < n;
    const uint32_t d = (uint32_t)(key[r] >> shift) & mask;
    // lanes of this group with the same digit: one ballot per digit bit; a lane keeps the lanes that agree with it
    const uint64_t vm = __ballot(valid);
    uint32_t mlo = (uint32_t)vm, mhi = (uint32_t)(vm >> 32);
    auto match_bit = [&](int b) {
      const uint32_t y = (uint32_t)__builtin_amdgcn_sbfe((int)d, b, 1); // all ones if the bit is set
      const uint64_t bal = __ballot(y != 0);
      mlo &= ~((uint32_t)bal ^ y);
      mhi &= ~((uint32_t)(bal >> 32) ^ y);
    };
    if (DBITS) {
#pragma unroll
      for (int b = 0; b < DBITS; b++) match_bit(b);
    } else {
      for (int b = 0; b < dbits; b++) match_bit(b);
    }
    const uint64_t m = ((uint64_t)mhi << 32) | mlo;
    // m: valid lanes of this group with the same digit (meaningless on invalid lanes)
    const uint32_t before = __popcll(m & ((1ull << lane) - 1ull));
    uint32_t prior = 0;
    if (valid) prior = cnt[w][d];
    __builtin_amdgcn_wave_barrier();
    const bool leader = valid && (m >> lane) == 1ull; // highest lane of the match group
    if (leader) cnt[w][d] = prior + before + 1;
    __builtin_amdgcn_wave_barrier();
    dig[r] = d;
    rnk[r] = prior + before;
  }
  __syncthreads();
  // wave-private counts -> offset of each wave's keys inside the bin; bin totals -> start of the bin in the tile
  {
    uint32_t tot[2] = {0, 0};
#pragma unroll
    for (int q = 0; q < 2; q++) {
      if (blo + q < bhi) {
        uint32_t run = 0;
#pragma unroll
        for (int ww = 0; ww < kWaves; ww++) {
          const uint32_t t = cnt[ww][blo + q];
          cnt[ww][blo + q] = run;
          run += t;
        }
        tot[q] = run;
      }
    }
    uint32_t total;
    uint32_t off = block_exclusive_scan<kSortBlock>(tot[0] + tot[1], sm, total);
#pragma unroll
    for (int q = 0; q < 2; q++) {
      if (blo + q < bhi) {
        bin_start[blo + q] = off;
        off += tot[q];
      }
    }
  }
  __syncthreads();
  // where every key goes in the tile sorted by digit
  uint32_t lp[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; r++) lp[r] = bin_start[dig[r]] + cnt[w][dig[r]] + rnk[r];
  __syncthreads(); // the counters are no longer needed: their area takes the sorted tile
#pragma unroll
  for (int r = 0; r < kRounds; r++) {
    const uint32_t idx = wbase + r * kWave + lane;
    if (idx < n) {
      skey[lp[r]] = key[r];
      sval[lp[r]] = val[r];
    }
  }
  __syncthreads();
  // neighbouring threads now hold neighbouring keys of a bin: the global stores of a bin are contiguous
  const uint32_t tile_n = min((uint32_t)kSortTile, n - tile * kSortTile);
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = k * kSortBlock + threadIdx.x;
    if (i < tile_n) {
      const K kk = skey[i];
      const uint32_t d = (uint32_t)(kk >> shift) & mask;
      const uint32_t pos = base[d] + (i - bin_start[d]);
      keys_out[pos] = kk;
      vals_out[pos] = sval[i];
    }
  }
}

} // namespace

template <typename K>
void radix_sort_positions(hipStream_t stream, const K *keys_in, uint32_t n, int bits, K *tmp_k0, K *tmp_k1,
                          uint32_t *tmp_v0, uint32_t *tmp_v1, uint32_t *vals_out, const SortScratch &scratch,
                          const K **keys_sorted, bool first_counts_done, int step_from, int step_to) {
  *keys_sorted = keys_in;
  if (n == 0) return;
  if (bits < 1) bits = 1;
  HCTR_CHECK(bits <= (int)sizeof(K) * 8, "sort key wider than its type");
  HCTR_CHECK(scratch.words != nullptr && n <= scratch.n_cap, "sort scratch too small");
  const uint32_t tiles = (uint32_t)sort_tiles(n);
  const uint32_t sgrid = (tiles + kXcds - 1) / kXcds * kXcds; // whole rounds over the XCDs
  uint32_t *counts = scratch.words;
  uint32_t *bin_total = scratch.words + (size_t)tiles * kSortMaxBins; // one row per piece of the scan
  const int passes = (bits + kSortMaxDigitBits - 1) / kSortMaxDigitBits;
  const bool self_scan = sort_items(n) == kSortItemsSmall && tiles <= kSelfScanTiles;
  const uint32_t pieces = sort_items(n) == kSortItemsLarge ? scan_chunks(tiles) : 1u;
  int shift = 0;
  const K *kin = keys_in;
  const uint32_t *vin = nullptr;
  K *ktmp[2] = {tmp_k0, tmp_k1};
  uint32_t *vtmp[2] = {tmp_v0, tmp_v1};
  for (int p = 0; p < passes; p++) {
    const int left = bits - shift;
    const int dbits = (left + (passes - p) - 1) / (passes - p);
    K *kout = ktmp[p & 1];
    uint32_t *vout = (p == passes - 1) ? vals_out : vtmp[p & 1];
    const uint32_t nb = 1u << dbits;
    auto wanted = [&](int kind) { return 3 * p + kind >= step_from && 3 * p + kind < step_to; };
    if (wanted(0) && (p > 0 || !first_counts_done)) {
#define CALL(I) \
  hipLaunchKernelGGL((digit_histogram<K, I>), dim3(tiles), dim3(kSortBlock), 0, stream, kin, n, shift, dbits, counts)
      HCTR_SORT_ITEMS_DISPATCH(n, CALL);
#undef CALL
    }
    if (wanted(1) && !self_scan)
      hipLaunchKernelGGL(scan_tiles, dim3((nb + kScanCols - 1) / kScanCols, pieces), dim3(kScanBlock), 0, stream, counts,
                         tiles, nb, bin_total);
    if (wanted(2)) {
#define CALL4(I, F, D, S)                                                                                     \
  hipLaunchKernelGGL((scatter<K, F, I, D, S>), dim3(sgrid), dim3(kSortBlock), 0, stream, kin, vin, kout, vout, n, \
                     shift, dbits, tiles, counts, bin_total, pieces)
#define CALL3(I, F, D)                                                                       \
  do {                                                                                       \
    if (self_scan && I == kSortItemsSmall) CALL4(I, F, D, (I == kSortItemsSmall ? 1 : 0));    \
    else if (pieces > 1 && I == kSortItemsLarge) CALL4(I, F, D, (I == kSortItemsLarge ? 2 : 0)); \
    else CALL4(I, F, D, 0);                                                                  \
  } while (0)
#define CALL2(I, F)                   \
  do {                                \
    switch (dbits) {                  \
      case 8: CALL3(I, F, 8); break;  \
      case 9: CALL3(I, F, 9); break;  \
      case 10: CALL3(I, F, 10); break; \
      default: CALL3(I, F, 0); break; \
    }                                 \
  } while (0)
#define CALL(I)                \
  do {                         \
    if (p == 0) CALL2(I, true); \
    else CALL2(I, false);      \
  } while (0)
      HCTR_SORT_ITEMS_DISPATCH(n, CALL);
#undef CALL
#undef CALL2
#undef CALL3
#undef CALL4
    }
    HCTR_HIP(hipGetLastError());
    kin = kout;
    vin = vout;
    shift += dbits;
  }
  *keys_sorted = kin;
}

template void radix_sort_positions<uint32_t>(hipStream_t, const uint32_t *, uint32_t, int, uint32_t *, uint32_t *,
                                             uint32_t *, uint32_t *, uint32_t *, const SortScratch &,
                                             const uint32_t **, bool, int, int);
template void radix_sort_positions<uint64_t>(hipStream_t, const uint64_t *, uint32_t, int, uint64_t *, uint64_t *,
                                             uint32_t *, uint32_t *, uint32_t *, const SortScratch &,
                                             const uint64_t **, bool, int, int);

} // namespace hctr
