// Stable LSD radix sort for gfx950, 64-lane wavefronts.
//
// One pass = three launches:
//   digit_histogram   per-block digit counts (LDS atomics) -> ghist[bin][block]
//   scan_bins         one block per digit value: exclusive scan of its row over the blocks + row total
//   scatter           per block: global base of every bin, stable rank of every key inside the block
//                     (wave-level match by ballots, wave-private LDS counters), the tile sorted by digit in
//                     LDS, then stores that are contiguous per bin
// Stability: a block's tile is split into 4 contiguous sub-tiles, one per wave; a wave walks its
// sub-tile 64 keys at a time in ascending position; inside such a group the rank among equal digits is
// the lane order.  Wave-private counters make the result independent of wave scheduling.
#include "radix_sort.h"

namespace hctr {
namespace {

constexpr int kWaves = kSortBlock / kWave;
constexpr int kSub = kSortTile / kWaves; // keys per wave
constexpr int kRounds = kSub / kWave;    // 64-key groups per wave

// kRuns: the keys are expected to come in long runs of equal digits (a sort key that is constant over most of the
// input).  A wave whose 64 keys share one digit then adds once instead of 64 times to the same LDS word.
template <typename K, bool kRuns>
__global__ __launch_bounds__(kSortBlock) void digit_histogram(const K *__restrict__ keys, uint32_t n, int shift,
                                                              int dbits, uint32_t *__restrict__ ghist,
                                                              uint32_t nblocks) {
  __shared__ uint32_t h[1 << kSortMaxDigitBits];
  const uint32_t nb = 1u << dbits, mask = nb - 1;
  for (uint32_t i = threadIdx.x; i < nb; i += kSortBlock) h[i] = 0;
  __syncthreads();
  const uint32_t base = blockIdx.x * kSortTile;
  K held[kSortItems]; // all loads of the thread first: they are in flight together
#pragma unroll
  for (int k = 0; k < kSortItems; k++) {
    uint32_t idx = base + k * kSortBlock + threadIdx.x;
    held[k] = idx < n ? keys[idx] : (K)0;
  }
#pragma unroll
  for (int k = 0; k < kSortItems; k++) {
    uint32_t idx = base + k * kSortBlock + threadIdx.x;
    const bool in = idx < n;
    const uint32_t d = in ? (uint32_t)(held[k] >> shift) & mask : 0;
    if (kRuns) {
      // lanes inside the input are a prefix of the wave, so lane 0 is inside whenever any lane is
      const unsigned long long act = __ballot(in);
      const uint32_t d0 = __builtin_amdgcn_readfirstlane(d);
      if (act != 0 && __ballot(in && d == d0) == act) {
        if (lane_id() == 0) atomicAdd(&h[d0], (uint32_t)__popcll(act));
        continue;
      }
    }
    if (in) atomicAdd(&h[d], 1u);
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < nb; i += kSortBlock) ghist[(size_t)i * nblocks + blockIdx.x] = h[i];
}

// grid = number of bins; block b scans row b of ghist in place (exclusive) and writes its total
__global__ __launch_bounds__(kSortBlock) void scan_bins(uint32_t *__restrict__ ghist, uint32_t nblocks,
                                                        uint32_t *__restrict__ bintot) {
  __shared__ uint32_t sm[kWaves + 1];
  uint32_t *row = ghist + (size_t)blockIdx.x * nblocks;
  const uint32_t per = (nblocks + kSortBlock - 1) / kSortBlock;
  const uint32_t lo = min(threadIdx.x * per, nblocks), hi = min(lo + per, nblocks);
  uint32_t s = 0;
  for (uint32_t i = lo; i < hi; i++) s += row[i];
  uint32_t total;
  uint32_t off = block_exclusive_scan<kSortBlock>(s, sm, total);
  for (uint32_t i = lo; i < hi; i++) {
    uint32_t v = row[i];
    row[i] = off;
    off += v;
  }
  if (threadIdx.x == 0) bintot[blockIdx.x] = total;
}

// kSmall: ghist holds the raw counts of a sort of few tiles (no scan kernel ran, bintot is unused): the block sums
// its bins over the blocks itself, which is cheaper than a launch when the blocks are few.
template <typename K, bool kFirst, bool kSmall = false>
__global__ __launch_bounds__(kSortBlock) void scatter(const K *__restrict__ keys_in, const uint32_t *__restrict__ vals_in,
                                                      K *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
                                                      uint32_t n, int shift, int dbits,
                                                      const uint32_t *__restrict__ ghist, uint32_t nblocks,
                                                      const uint32_t *__restrict__ bintot) {
  __shared__ uint32_t cnt[kWaves][1 << kSortMaxDigitBits];
  __shared__ uint32_t base[1 << kSortMaxDigitBits];      // global position of the bin's first key of this block
  __shared__ uint32_t bin_start[1 << kSortMaxDigitBits]; // position of the bin inside the block's sorted tile
  __shared__ K skey[kSortTile];
  __shared__ uint32_t sval[kSortTile];
  __shared__ uint32_t sm[kWaves + 1];
  const uint32_t nb = 1u << dbits, mask = nb - 1;
  const int w = threadIdx.x / kWave;
  const unsigned lane = lane_id();
  const uint32_t per = (nb + kSortBlock - 1) / kSortBlock; // consecutive bins per thread in the two bin scans
  const uint32_t blo = min(threadIdx.x * per, nb), bhi = min(blo + per, nb);

  // global base of each bin for this block: sum of the totals of lower bins + this bin's lower blocks
  if (kSmall) {
    uint32_t s = 0;
    for (uint32_t i = blo; i < bhi; i++) {
      const uint32_t *row = ghist + (size_t)i * nblocks;
      uint32_t lower = 0, all = 0;
      for (uint32_t j = 0; j < nblocks; j++) {
        const uint32_t v = row[j];
        lower += j < blockIdx.x ? v : 0u;
        all += v;
      }
      base[i] = lower;      // completed below
      bin_start[i] = all;   // the bin's total, parked here until the scan is through
      s += all;
    }
    uint32_t total;
    uint32_t off = block_exclusive_scan<kSortBlock>(s, sm, total);
    for (uint32_t i = blo; i < bhi; i++) {
      base[i] += off;
      off += bin_start[i];
    }
  } else {
    uint32_t s = 0;
    for (uint32_t i = blo; i < bhi; i++) s += bintot[i];
    uint32_t total;
    uint32_t off = block_exclusive_scan<kSortBlock>(s, sm, total);
    for (uint32_t i = blo; i < bhi; i++) {
      base[i] = off + ghist[(size_t)i * nblocks + blockIdx.x];
      off += bintot[i];
    }
  }
  for (uint32_t i = threadIdx.x; i < kWaves * nb; i += kSortBlock) cnt[i / nb][i % nb] = 0;
  __syncthreads();

  // stable rank of every key among the keys of its wave with the same digit
  K key[kRounds];
  uint32_t val[kRounds];
  uint32_t dig[kRounds];
  uint32_t rnk[kRounds];
  const uint32_t wbase = blockIdx.x * kSortTile + w * kSub;
#pragma unroll
  for (int r = 0; r < kRounds; r++) {
    const uint32_t idx = wbase + r * kWave + lane;
    const bool valid = idx < n;
    // a pass reads its input once
    key[r] = valid ? load_once(&keys_in[idx]) : (K)0;
    val[r] = kFirst ? idx : (valid ? load_once(&vals_in[idx]) : 0u);
  }
#pragma unroll
  for (int r = 0; r < kRounds; r++) {
    const uint32_t idx = wbase + r * kWave + lane;
    const bool valid = idx < n;
    const uint32_t d = (uint32_t)(key[r] >> shift) & mask;
    uint64_t m = __ballot(valid);
    for (int b = 0; b < dbits; b++) {
      const bool bit = (d >> b) & 1u;
      const uint64_t bal = __ballot(bit);
      m &= bit ? bal : ~bal;
    }
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
    uint32_t s = 0;
    for (uint32_t i = blo; i < bhi; i++) {
      uint32_t run = 0;
#pragma unroll
      for (int ww = 0; ww < kWaves; ww++) {
        const uint32_t t = cnt[ww][i];
        cnt[ww][i] = run;
        run += t;
      }
      bin_start[i] = run; // total of the bin for now
      s += run;
    }
    uint32_t total;
    uint32_t off = block_exclusive_scan<kSortBlock>(s, sm, total);
    for (uint32_t i = blo; i < bhi; i++) {
      const uint32_t t = bin_start[i];
      bin_start[i] = off;
      off += t;
    }
  }
  __syncthreads();
  // the tile, sorted by digit, in LDS
#pragma unroll
  for (int r = 0; r < kRounds; r++) {
    const uint32_t idx = wbase + r * kWave + lane;
    if (idx < n) {
      const uint32_t lp = bin_start[dig[r]] + cnt[w][dig[r]] + rnk[r];
      skey[lp] = key[r];
      sval[lp] = val[r];
    }
  }
  __syncthreads();
  // neighbouring threads now hold neighbouring keys of a bin: the global stores of a bin are contiguous
  const uint32_t tile_n = min((uint32_t)kSortTile, n - blockIdx.x * kSortTile);
#pragma unroll
  for (int k = 0; k < kSortItems; k++) {
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
                          const K **keys_sorted, bool first_hist_done, bool long_runs) {
  *keys_sorted = keys_in;
  if (n == 0) return;
  if (bits < 1) bits = 1;
  HCTR_CHECK(bits <= (int)sizeof(K) * 8, "sort key wider than its type");
  const uint32_t nblocks = (uint32_t)sort_blocks(n);
  HCTR_CHECK(nblocks <= scratch.blocks_cap, "sort scratch too small");
  const int passes = (bits + kSortMaxDigitBits - 1) / kSortMaxDigitBits;
  int shift = 0;
  const K *kin = keys_in;
  const uint32_t *vin = nullptr;
  K *ktmp[2] = {tmp_k0, tmp_k1};
  uint32_t *vtmp[2] = {tmp_v0, tmp_v1};
  const bool small = nblocks <= kSmallSortBlocks;
  for (int p = 0; p < passes; p++) {
    const int left = bits - shift;
    const int dbits = (left + (passes - p) - 1) / (passes - p);
    K *kout = ktmp[p & 1];
    uint32_t *vout = (p == passes - 1) ? vals_out : vtmp[p & 1];
    const uint32_t nb = 1u << dbits;
    if (p > 0 || !first_hist_done) {
      if (long_runs)
        hipLaunchKernelGGL((digit_histogram<K, true>), dim3(nblocks), dim3(kSortBlock), 0, stream, kin, n, shift,
                           dbits, scratch.ghist, nblocks);
      else
        hipLaunchKernelGGL((digit_histogram<K, false>), dim3(nblocks), dim3(kSortBlock), 0, stream, kin, n, shift,
                           dbits, scratch.ghist, nblocks);
    }
    if (small) { // few tiles: the blocks of the scatter scan the raw counts themselves
      if (p == 0)
        hipLaunchKernelGGL((scatter<K, true, true>), dim3(nblocks), dim3(kSortBlock), 0, stream, kin, vin, kout, vout, n,
                           shift, dbits, scratch.ghist, nblocks, scratch.bintot);
      else
        hipLaunchKernelGGL((scatter<K, false, true>), dim3(nblocks), dim3(kSortBlock), 0, stream, kin, vin, kout, vout,
                           n, shift, dbits, scratch.ghist, nblocks, scratch.bintot);
    } else {
      hipLaunchKernelGGL(scan_bins, dim3(nb), dim3(kSortBlock), 0, stream, scratch.ghist, nblocks, scratch.bintot);
      if (p == 0)
        hipLaunchKernelGGL((scatter<K, true>), dim3(nblocks), dim3(kSortBlock), 0, stream, kin, vin, kout, vout, n,
                           shift, dbits, scratch.ghist, nblocks, scratch.bintot);
      else
        hipLaunchKernelGGL((scatter<K, false>), dim3(nblocks), dim3(kSortBlock), 0, stream, kin, vin, kout, vout, n,
                           shift, dbits, scratch.ghist, nblocks, scratch.bintot);
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
                                             const uint32_t **, bool, bool);
template void radix_sort_positions<uint64_t>(hipStream_t, const uint64_t *, uint32_t, int, uint64_t *, uint64_t *,
                                             uint32_t *, uint32_t *, uint32_t *, const SortScratch &,
                                             const uint64_t **, bool, bool);

} // namespace hctr
