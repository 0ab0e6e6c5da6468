// Tile-sorted passes of the key sort for gfx950 (see tile_sort.h): passes + 1 launches, 64-lane wavefronts, no global
// atomics, no block that waits for another.
//
// Data between two launches: the (key, position) pairs cut into tiles of ITEMS * kSortBlock pairs in the order the passes
// so far established, every tile sorted stably by the next digit d, and table[b][tile] = place of the first pair of the
// tile with digit b (two-byte entries: a tile holds at most 8192 pairs; a column, i.e. one digit value over all tiles, is
// contiguous).  The place of a pair in the order by d follows:
// pairs with a smaller digit first (their number is the sum of column d of the table), then the pairs with digit d of the
// earlier tiles, then the pair's place among the tile's pairs with digit d -- (digit, tile) pieces are contiguous both in
// their tile and in the new order, so block o, which produces positions [o * tile, (o + 1) * tile) of the new order, finds
// the pieces that overlap its range and copies them.
#include "tile_sort.h"

namespace hctr {
namespace {

constexpr int kWaves = kSortBlock / kWave;
constexpr int cmax(int a, int b) { return a > b ? a : b; }
static_assert(kSortMaxBins <= 2 * kSortBlock, "a thread owns at most two bins");
static_assert(kTileItemsMax * kSortBlock <= 65535, "table entries are two bytes");

template <typename K, int ITEMS> struct TileShape {
  static constexpr int kTile = ITEMS * kSortBlock; // pairs per tile
  static constexpr int kSub = ITEMS * kWave;       // pairs per wave: wave w holds elements w * kSub + r * 64 + lane
  // one LDS area, used for one thing after the other: the segment starts of the regrouping, the wave-private digit
  // counters, the tile sorted by digit
  static constexpr int kCntWords = kWaves * kSortMaxBins;
  static constexpr int kPermWords = kTile * (int)(sizeof(K) / 4 + 1);
  static constexpr int kGatherWords = 2 * kTile;
  static constexpr int kAreaWords = cmax(cmax(kCntWords, kPermWords), kGatherWords);
};

// Sorts the block's tile by one digit, stably.  key / val: element e = w * kSub + r * 64 + lane of the tile in registers
// (e < tile_n holds a pair).  `area` must be free (a barrier behind its last use).  On return the tile lies sorted in
// area (keys, then positions) and bin_start[b] is the place of the first pair with digit b; a barrier has been passed.
// A wave ranks 64 keys at a time by one ballot per digit bit into wave-private counters: no atomics, and the result
// does not depend on how the waves are scheduled.
// The digit of a key is ((key >> shift) & field) - bias, a value below 1 << dbits (a block that knows its keys only
// take a few neighbouring digit values ranks them with as many ballots as those values need bits).
template <typename K, int ITEMS, int DBITS>
__device__ __forceinline__ void tile_sort_by_digit(const K (&key)[ITEMS], const uint32_t (&val)[ITEMS], uint32_t tile_n,
                                                   int shift, int dbits, uint32_t *area, uint32_t *bin_start,
                                                   uint32_t *sm, uint32_t field = ~0u, uint32_t bias = 0) {
  using S = TileShape<K, ITEMS>;
  uint32_t(*cnt)[kSortMaxBins] = (uint32_t(*)[kSortMaxBins])area;
  K *skey = (K *)area;
  uint32_t *sval = area + S::kTile * (sizeof(K) / 4);
  const uint32_t nb = 1u << dbits, mask = nb - 1;
  const int w = threadIdx.x / kWave;
  const unsigned lane = lane_id();
  const uint32_t per = nb > (uint32_t)kSortBlock ? nb / kSortBlock : 1u;
  const uint32_t blo = min(threadIdx.x * per, nb), bhi = min(blo + per, nb);
  for (uint32_t i = threadIdx.x; i < kWaves * nb; i += kSortBlock) cnt[i >> dbits][i & mask] = 0;
  __syncthreads();
  uint32_t dig[ITEMS], rnk[ITEMS];
#pragma unroll
  for (int r = 0; r < ITEMS; r++) {
    const uint32_t e = w * S::kSub + r * kWave + lane;
    const bool valid = e < tile_n;
    const uint32_t d = (((uint32_t)(key[r] >> shift) & field) - bias) & mask;
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
  uint32_t lp[ITEMS];
#pragma unroll
  for (int r = 0; r < ITEMS; r++) lp[r] = bin_start[dig[r]] + cnt[w][dig[r]] + rnk[r];
  __syncthreads(); // the counters are no longer needed: their area takes the sorted tile
#pragma unroll
  for (int r = 0; r < ITEMS; r++) {
    const uint32_t e = w * S::kSub + r * kWave + lane;
    if (e < tile_n) {
      skey[lp[r]] = key[r];
      sval[lp[r]] = val[r];
    }
  }
  __syncthreads();
}

// the sorted tile to global memory (whole-line stores: the tile is contiguous) and its column of the table
template <typename K, int ITEMS>
__device__ __forceinline__ void store_sorted_tile(const uint32_t *area, const uint32_t *bin_start, uint32_t tile,
                                                  uint32_t tile_n, int dbits, uint32_t pitch, K *__restrict__ out_keys,
                                                  uint32_t *__restrict__ out_vals, uint16_t *__restrict__ table) {
  using S = TileShape<K, ITEMS>;
  const K *skey = (const K *)area;
  const uint32_t *sval = area + S::kTile * (sizeof(K) / 4);
  const size_t lo = (size_t)tile * S::kTile;
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = k * kSortBlock + threadIdx.x;
    if (i < tile_n) {
      out_keys[lo + i] = skey[i];
      out_vals[lo + i] = sval[i];
    }
  }
  const uint32_t nb = 1u << dbits;
  for (uint32_t b = threadIdx.x; b < nb; b += kSortBlock) table[(size_t)b * pitch + tile] = (uint16_t)bin_start[b];
}

// Launch 0: ids -> sort keys (owner << id_bits | id), the range check, the reset of the batch's run counters, and the
// tile sorted by the first digit.  This is the one kernel that reads the caller's buffer: the call may return when it
// is through.  (csrc/core/preprocess.cu:11-20 builds the reference's sort key.)
// kFromKeys: the sort keys have been made already (make_keys, for a caller that wants its buffer back sooner than a
// tile is sorted): `ids` then points to them, and nothing is checked or reset here.
template <typename K, int ITEMS, int DBITS, bool kFromKeys>
__global__ __launch_bounds__(kSortBlock) void keys_tile_sort(const void *__restrict__ ids_or_keys, uint32_t n,
                                                              uint64_t id_max, int id_bits, int nrank,
                                                              const worker_t *__restrict__ root, uint32_t *__restrict__ err,
                                                              uint32_t *__restrict__ nlong, int dbits, uint32_t pitch,
                                                              K *__restrict__ out_keys, uint32_t *__restrict__ out_vals,
                                                              uint16_t *__restrict__ table, bool ids32,
                                                              K *__restrict__ keys_out) {
  using S = TileShape<K, ITEMS>;
  __shared__ __align__(16) uint32_t area[S::kAreaWords];
  __shared__ uint32_t bin_start[kSortMaxBins];
  __shared__ uint32_t sm[kWaves + 1];
  const uint32_t tile = blockIdx.x, tile_lo = tile * S::kTile;
  const uint32_t tile_n = min((uint32_t)S::kTile, n - tile_lo);
  const int w = threadIdx.x / kWave;
  const unsigned lane = lane_id();
  K key[ITEMS];
  uint32_t val[ITEMS];
  if (kFromKeys) {
    const K *__restrict__ keys = (const K *)ids_or_keys;
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      const uint32_t e = w * S::kSub + r * kWave + lane;
      key[r] = e < tile_n ? keys[tile_lo + e] : (K)0;
      val[r] = tile_lo + e;
    }
  } else {
    const index_t *__restrict__ ids = (const index_t *)ids_or_keys;
    if (blockIdx.x == 0 && threadIdx.x < kRunCounters && nlong) nlong[threadIdx.x] = 0; // counters of this batch
    uint64_t id[ITEMS];
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      const uint32_t e = w * S::kSub + r * kWave + lane;
      // the caller's ids are read here and nowhere else (ids32: as narrowed on their way from pageable host memory)
      id[r] = e >= tile_n ? 0 : ids32 ? (uint64_t)load_once(&((const uint32_t *)ids)[tile_lo + e]) : (uint64_t)load_once(&ids[tile_lo + e]);
    }
    bool bad = false;
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      const uint32_t e = w * S::kSub + r * kWave + lane;
      if (e < tile_n && id[r] >= id_max) { // also catches negative ids
        bad = true;
        id[r] = 0;
      }
    }
    if (bad) atomicOr(err, 1u);
    uint64_t owner[ITEMS];
#pragma unroll
    for (int r = 0; r < ITEMS; r++) owner[r] = nrank > 1 ? root[id[r]] : 0;
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      key[r] = (K)((owner[r] << id_bits) | id[r]);
      val[r] = tile_lo + w * S::kSub + r * kWave + lane;
      // the sort keys in batch order as well, for a caller that works on the batch before it is sorted (optional)
      if (keys_out && w * S::kSub + r * kWave + lane < tile_n) keys_out[val[r]] = key[r];
    }
  }
  tile_sort_by_digit<K, ITEMS, DBITS>(key, val, tile_n, 0, dbits, area, bin_start, sm);
  store_sorted_tile<K, ITEMS>(area, bin_start, tile, tile_n, dbits, pitch, out_keys, out_vals, table);
}

// Sums of kCols table columns (kCols a power of two <= 64) into LDS words acc[0..kCols): lane l of every wave adds up
// column col(l % kCols); the threads that share a column split its tiles, 8 consecutive tiles (one 16-byte load) at a
// time, request all their loads before they use the first, and add one partial sum each to the column's word (lanes of
// one instruction add to different words).
template <int kCols, int kMax, typename ColumnOf>
__device__ __forceinline__ void add_columns(const uint16_t *__restrict__ table, uint32_t pitch, uint32_t tiles,
                                            uint32_t nb, uint32_t *__restrict__ acc, ColumnOf col) {
  constexpr int kShare = kSortBlock / kCols; // threads per column
  const uint32_t groups = pitch / 8;         // 16-byte groups of a column
  const uint32_t c = threadIdx.x % kCols, part = threadIdx.x / kCols, b = col(c);
  if (b >= nb) return;
  uint4 v[kMax];
#pragma unroll
  for (int a = 0; a < kMax; a++) {
    const uint32_t g = part + a * kShare;
    v[a] = make_uint4(0, 0, 0, 0);
    if (g < groups) v[a] = *(const uint4 *)(table + (size_t)b * pitch + g * 8);
  }
  uint32_t s = 0;
#pragma unroll
  for (int a = 0; a < kMax; a++) {
    const uint32_t g = part + a * kShare;
    if (g >= groups) continue;
    const uint32_t wd[4] = {v[a].x, v[a].y, v[a].z, v[a].w};
#pragma unroll
    for (int h = 0; h < 4; h++) {
      const uint32_t t = g * 8 + 2 * h;
      s += (t < tiles ? wd[h] & 0xffffu : 0u) + (t + 1 < tiles ? wd[h] >> 16 : 0u); // the padding is not initialised
    }
  }
  atomicAdd(&acc[c], s); // LDS
}

constexpr uint32_t kCoarse = 32;    // digit values per step of the first round of the column search
static_assert((kTileSortMaxTiles + 7) / 8 <= 2 * (kSortBlock / kCoarse) && (kTileSortMaxTiles + 7) / 8 <= 4 * (kSortBlock / (2 * kCoarse)) &&
                  kSortMaxBins <= kCoarse * kCoarse,
              "two loads per thread cover a column in the coarse round, four in the fine round");


// Launches 1..P.  Block o produces positions [o * tile, (o + 1) * tile) of the order by the digit the input tiles are
// sorted by (shift_in, dbits_in, table_in), then either sorts them by the next digit for the following pass (kLast
// false) or writes them out as the final result with the head counts of its chunks (kLast true).
//
// The block's positions hold the pairs with digit values b_lo..b_hi (without those of b_lo before its first position
// and those of b_hi behind its last).  Inside an input tile these pairs are ONE contiguous segment, because the tile is
// sorted by that digit: the block fetches one segment per tile -- whole lines even where a single (digit, tile) piece
// is a pair or two -- and, holding them in tile order, sorts them stably by the digit, which is the order wanted; the
// few digit values of a block take few ballots per key.
template <typename K, int ITEMS, int DBITS, bool kLast>
__global__ __launch_bounds__(kSortBlock) void regroup(const K *__restrict__ in_keys, const uint32_t *__restrict__ in_vals,
                                                       const uint16_t *__restrict__ table_in, int shift_in, int dbits_in,
                                                       uint32_t n, uint32_t tiles, uint32_t pitch,
                                                       K *__restrict__ out_keys, uint32_t *__restrict__ out_vals,
                                                       uint16_t *__restrict__ table_out, int shift, int dbits,
                                                       uint32_t *__restrict__ head_inner, K *__restrict__ head_first,
                                                       K *__restrict__ head_last) {
  using S = TileShape<K, ITEMS>;
  __shared__ __align__(16) uint32_t area[S::kAreaWords];
  __shared__ uint32_t bin_start[kSortMaxBins];
  __shared__ uint32_t sm[kWaves + 1];
  __shared__ uint32_t coarse[kCoarse], fine[2 * kCoarse];
  __shared__ uint32_t found[6];
  __shared__ uint32_t wmax[kWaves];
  const uint32_t tile = blockIdx.x;
  const uint32_t p0 = tile * S::kTile, tile_n = min((uint32_t)S::kTile, n - p0), p1 = p0 + tile_n;
  const uint32_t nb = 1u << dbits_in;
  const int w = threadIdx.x / kWave;
  const unsigned lane = lane_id();

  // ---- The digit values of the block's first and last position.  Digit value b starts at the sum of column b of the
  // table (the entries are prefix sums over the digit values inside a tile), and these starts ascend with b: two rounds
  // of column sums find both values, first every 32nd column, then the 32 columns behind the coarse hits.
  const uint32_t n_coarse = (nb + kCoarse - 1) / kCoarse; // <= 32
  if (threadIdx.x < kCoarse) coarse[threadIdx.x] = 0;
  if (threadIdx.x < 2 * kCoarse) fine[threadIdx.x] = 0;
  __syncthreads();
  add_columns<kCoarse, 2>(table_in, pitch, tiles, nb, coarse, [](uint32_t c) { return c * kCoarse; });
  __syncthreads();
  if (threadIdx.x < kWave) {
    const bool in = lane < n_coarse;
    const uint32_t v = in ? coarse[lane] : 0u;
    // coarse[0] = 0 <= p0 < p1: both counts are at least one
    const uint32_t c_lo = __popcll(__ballot(in && v <= p0)) - 1, c_hi = __popcll(__ballot(in && v < p1)) - 1;
    if (lane == 0) {
      found[0] = c_lo;
      found[1] = c_hi;
    }
  }
  __syncthreads();
  {
    const uint32_t c_lo = found[0], c_hi = found[1];
    add_columns<2 * kCoarse, 4>(table_in, pitch, tiles, nb, fine,
                                [=](uint32_t c) { return (c < kCoarse ? c_lo : c_hi) * kCoarse + (c & (kCoarse - 1)); });
    __syncthreads();
    if (threadIdx.x < kWave) {
      const bool in_lo = lane < kCoarse && c_lo * kCoarse + lane < nb, in_hi = lane < kCoarse && c_hi * kCoarse + lane < nb;
      const uint32_t v_lo = in_lo ? fine[lane] : 0u, v_hi = in_hi ? fine[kCoarse + lane] : 0u;
      const uint32_t f_lo = __popcll(__ballot(in_lo && v_lo <= p0)) - 1, f_hi = __popcll(__ballot(in_hi && v_hi < p1)) - 1;
      if (lane == 0) {
        found[2] = c_lo * kCoarse + f_lo;   // digit value of the block's first position
        found[3] = c_hi * kCoarse + f_hi;   // ... and of its last
        found[4] = fine[f_lo];              // where the first digit value starts
        found[5] = fine[kCoarse + f_hi];    // where the last one starts
      }
    }
  }
  uint32_t *marker = area;            // [tile] place + 1 at the places where a tile's segment starts, else 0
  uint32_t *srcat = area + S::kTile;  // [tile] at such a place: where the segment's first pair lies in the input
#pragma unroll
  for (int k = 0; k < ITEMS; k++) marker[k * kSortBlock + threadIdx.x] = 0;
  __syncthreads();
  const uint32_t b_lo = found[2], b_hi = found[3];
  {
    // thread t: the segment of input tile t.  Of digit value b_lo the block takes the pairs from its first position on,
    // counted over the tiles in order; of b_hi those up to its last position.
    const uint32_t t = threadIdx.x;
    const bool in = t < tiles;
    const uint32_t size_t_ = in ? min((uint32_t)S::kTile, n - t * S::kTile) : 0u;
    uint32_t a = 0, a1 = 0, h = 0, h1 = 0;
    if (in) {
      a = table_in[(size_t)b_lo * pitch + t];
      a1 = b_lo + 1 < nb ? (uint32_t)table_in[(size_t)(b_lo + 1) * pitch + t] : size_t_;
      h = table_in[(size_t)b_hi * pitch + t];
      h1 = b_hi + 1 < nb ? (uint32_t)table_in[(size_t)(b_hi + 1) * pitch + t] : size_t_;
    }
    uint32_t total;
    const uint32_t x_lo = block_exclusive_scan<kSortBlock>(a1 - a, sm, total); // pairs with b_lo in the tiles before
    const uint32_t x_hi = block_exclusive_scan<kSortBlock>(h1 - h, sm, total);
    const uint32_t skip = p0 - found[4];  // pairs with b_lo that lie before the block's first position
    const uint32_t keep = p1 - found[5];  // pairs with b_hi up to the block's last position
    const uint32_t front = min(a1 - a, skip > x_lo ? skip - x_lo : 0u);
    const uint32_t back = min(h1 - h, keep > x_hi ? keep - x_hi : 0u);
    const uint32_t seg_lo = a + front, seg_hi = h + back;
    const uint32_t len = in && seg_hi > seg_lo ? seg_hi - seg_lo : 0u;
    const uint32_t dst = block_exclusive_scan<kSortBlock>(len, sm, total);
    if (len) {
      marker[dst] = dst + 1;
      srcat[dst] = t * S::kTile + seg_lo;
    }
  }
  __syncthreads();
  // ---- every place finds the segment it lies in (the last segment start at or before it) and fetches its pair
  K key[ITEMS];
  uint32_t val[ITEMS];
  {
    uint32_t m[ITEMS];
#pragma unroll
    for (int r = 0; r < ITEMS; r++) m[r] = marker[w * S::kSub + r * kWave + lane];
    // the last segment start in this wave's share, for the waves behind it (the marks ascend with the place)
    uint32_t last_mark = 0;
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      const uint64_t mask = __ballot(m[r] != 0);
      if (mask) last_mark = __builtin_amdgcn_readlane(m[r], 63 - __clzll(mask));
    }
    if (lane == 0) wmax[w] = last_mark;
    __syncthreads();
    uint32_t carry = 0; // last segment start before the places this wave has looked at
    for (int ww = 0; ww < w; ww++) carry = max(carry, wmax[ww]);
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      const uint32_t e = w * S::kSub + r * kWave + lane;
      const uint64_t mask = __ballot(m[r] != 0);
      const uint64_t below = mask & (~0ull >> (63 - lane)); // segment starts at this lane or before it in the round
      const uint32_t got = __shfl(m[r], below ? 63 - __clzll(below) : 0, kWave);
      const uint32_t v = below ? got : carry;
      if (mask) carry = __builtin_amdgcn_readlane(m[r], 63 - __clzll(mask));
      key[r] = (K)0;
      val[r] = 0;
      if (e < tile_n) {
        const uint32_t s = v - 1;
        const uint32_t from = srcat[s] + (e - s);
        key[r] = load_once(&in_keys[from]); // a pass reads its input once
        val[r] = load_once(&in_vals[from]);
      }
    }
  }
  if (b_hi != b_lo) {
    // tile order -> order by the digit (stable: tiles, and the pairs of a tile, keep their order inside a digit value)
    const int bits = 32 - __clz(b_hi - b_lo);
    __syncthreads(); // the segment starts are dead: the area takes the digit counters
    tile_sort_by_digit<K, ITEMS, 0>(key, val, tile_n, shift_in, bits, area, bin_start, sm, nb - 1, b_lo);
    const K *skey = (const K *)area;
    const uint32_t *sval = area + S::kTile * (sizeof(K) / 4);
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
      const uint32_t e = w * S::kSub + r * kWave + lane;
      if (e < tile_n) {
        key[r] = skey[e];
        val[r] = sval[e];
      }
    }
  }
  if (!kLast) {
    __syncthreads(); // what the area held is dead: it takes the digit counters
    tile_sort_by_digit<K, ITEMS, DBITS>(key, val, tile_n, shift, dbits, area, bin_start, sm);
    store_sorted_tile<K, ITEMS>(area, bin_start, tile, tile_n, dbits, pitch, out_keys, out_vals, table_out);
    return;
  }
  // ---- the final order: sorted keys, sorted positions, and per chunk (this wave's share) what counts unique keys
  const uint32_t sub_lo = w * S::kSub;
  if (sub_lo >= tile_n) return;
  const uint32_t sub_n = min((uint32_t)S::kSub, tile_n - sub_lo);
  uint32_t heads = 0;
  K before = (K)0; // key of lane 63 of the round before
#pragma unroll
  for (int r = 0; r < ITEMS; r++) {
    const uint32_t e = r * kWave + lane; // place in the chunk
    const bool valid = e < sub_n;
    if (valid) {
      out_keys[p0 + sub_lo + e] = key[r];
      out_vals[p0 + sub_lo + e] = val[r];
    }
    K prev = (K)__shfl_up(key[r], 1, kWave);
    if (lane == 0) prev = before;
    before = (K)__shfl(key[r], kWave - 1, kWave);
    heads += __popcll(__ballot(valid && e > 0 && key[r] != prev));
    if (valid && e == sub_n - 1) head_last[tile * kWaves + w] = key[r];
  }
  if (lane == 0) {
    head_inner[tile * kWaves + w] = heads;
    head_first[tile * kWaves + w] = key[0];
  }
}

// digit widths and shifts of the passes: the bits are split evenly, as radix_sort_positions does
struct DigitPlan {
  int passes;
  int dbits[64], shift[64];
};
DigitPlan plan_digits(const KeyLayout &kl) {
  DigitPlan p;
  const int bits = kl.total_bits < 1 ? 1 : kl.total_bits;
  const int widest = kl.max_digit_bits >= 1 && kl.max_digit_bits <= kSortMaxDigitBits ? kl.max_digit_bits : kSortMaxDigitBits;
  p.passes = (bits + widest - 1) / widest;
  int shift = 0;
  for (int i = 0; i < p.passes; i++) {
    const int left = bits - shift;
    p.dbits[i] = (left + (p.passes - i) - 1) / (p.passes - i);
    p.shift[i] = shift;
    shift += p.dbits[i];
  }
  return p;
}

} // namespace

// expands CALL(K, ITEMS, DBITS) for the key type, the tile shape of n keys and the digit width
#define HCTR_TILE_SORT_DISPATCH(wide, n, dbits, CALL)                                  \
  do {                                                                                 \
    const int items__ = ::hctr::tile_items(n);                                         \
    const int db__ = (dbits) == 8 || (dbits) == 9 || (dbits) == 10 ? (dbits) : 0;      \
    if (wide) HCTR_TILE_SORT_DISPATCH_I(uint64_t, items__, db__, CALL);                \
    else HCTR_TILE_SORT_DISPATCH_I(uint32_t, items__, db__, CALL);                     \
  } while (0)
#define HCTR_TILE_SORT_DISPATCH_I(K, items, db, CALL)             \
  do {                                                            \
    switch (items) {                                              \
      case 2: HCTR_TILE_SORT_DISPATCH_D(K, 2, db, CALL); break;   \
      case 4: HCTR_TILE_SORT_DISPATCH_D(K, 4, db, CALL); break;   \
      case 8: HCTR_TILE_SORT_DISPATCH_D(K, 8, db, CALL); break;   \
      case 13: HCTR_TILE_SORT_DISPATCH_D(K, 13, db, CALL); break; \
      default: HCTR_TILE_SORT_DISPATCH_D(K, 16, db, CALL); break; \
    }                                                             \
  } while (0)
#define HCTR_TILE_SORT_DISPATCH_D(K, I, db, CALL) \
  do {                                            \
    switch (db) {                                 \
      case 8: CALL(K, I, 8); break;               \
      case 9: CALL(K, I, 9); break;               \
      case 10: CALL(K, I, 10); break;             \
      default: CALL(K, I, 0); break;              \
    }                                             \
  } while (0)

void launch_tile_sort_keys(hipStream_t s, const TableView &t, const KeyLayout &kl, const index_t *ids,
                           const void *made_keys, uint32_t n, const TileSortBuffers &b, uint32_t *err, uint32_t *nlong,
                           bool ids32, void *keys_out) {
  if (!n) return;
  HCTR_CHECK(!ids32 || t.id_max <= 0xffffffffull, "internal: narrowed ids and a table of 2^32 rows or more");
  HCTR_CHECK(tile_sort_possible(n), "internal: batch too large for the tile-sorted passes");
  const DigitPlan p = plan_digits(kl);
  const unsigned tiles = (unsigned)tile_count(n), pitch = (unsigned)tile_table_pitch(n);
  uint16_t *table0 = (uint16_t *)b.tables;
#define CALL(K, I, D)                                                                                                 \
  do {                                                                                                                \
    if (made_keys)                                                                                                    \
      hipLaunchKernelGGL((keys_tile_sort<K, I, D, true>), dim3(tiles), dim3(kSortBlock), 0, s, made_keys, n, t.id_max, \
                         kl.id_bits, t.nrank, t.root, err, nlong, p.dbits[0], pitch, (K *)b.keys[0], b.vals[0], table0, \
                         false, (K *)nullptr);                                                                        \
    else                                                                                                              \
      hipLaunchKernelGGL((keys_tile_sort<K, I, D, false>), dim3(tiles), dim3(kSortBlock), 0, s, (const void *)ids, n, \
                         t.id_max, kl.id_bits, t.nrank, t.root, err, nlong, p.dbits[0], pitch, (K *)b.keys[0],        \
                         b.vals[0], table0, ids32, (K *)keys_out);                                                    \
  } while (0)
  HCTR_TILE_SORT_DISPATCH(kl.wide, n, p.dbits[0], CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

int launch_tile_sort_passes(hipStream_t s, const KeyLayout &kl, uint32_t n, const TileSortBuffers &b,
                            uint32_t *sorted_arg, const HeadChunks &heads, const void **sorted_keys, int from, int to) {
  const DigitPlan p = plan_digits(kl);
  *sorted_keys = b.keys[p.passes & 1];
  if (!n) return p.passes;
  const unsigned tiles = (unsigned)tile_count(n), pitch = (unsigned)tile_table_pitch(n);
  HCTR_CHECK(heads.chunk == (uint32_t)tile_items(n) * kWave, "internal: head chunks do not match the tile shape");
  uint16_t *table[2] = {(uint16_t *)b.tables, (uint16_t *)b.tables + (size_t)pitch * kSortMaxBins};
  for (int j = std::max(from, 1); j <= p.passes && j < to; j++) {
    const int in = (j - 1) & 1, out = j & 1;
    if (j < p.passes) {
#define CALL(K, I, D)                                                                                                   \
  hipLaunchKernelGGL((regroup<K, I, D, false>), dim3(tiles), dim3(kSortBlock), 0, s, (const K *)b.keys[in], b.vals[in], \
                     table[in], p.shift[j - 1], p.dbits[j - 1], n, tiles, pitch, (K *)b.keys[out], b.vals[out],         \
                     table[out], p.shift[j], p.dbits[j], (uint32_t *)nullptr, (K *)nullptr, (K *)nullptr)
      HCTR_TILE_SORT_DISPATCH(kl.wide, n, p.dbits[j], CALL);
#undef CALL
    } else {
#define CALL(K, I, D)                                                                                                  \
  hipLaunchKernelGGL((regroup<K, I, 0, true>), dim3(tiles), dim3(kSortBlock), 0, s, (const K *)b.keys[in], b.vals[in], \
                     table[in], p.shift[j - 1], p.dbits[j - 1], n, tiles, pitch, (K *)b.keys[out], sorted_arg,         \
                     (uint16_t *)nullptr, 0, 0, heads.inner, (K *)heads.first, (K *)heads.last)
      HCTR_TILE_SORT_DISPATCH(kl.wide, n, 0, CALL);
#undef CALL
    }
  }
  HCTR_HIP(hipGetLastError());
  return p.passes;
}

} // namespace hctr
