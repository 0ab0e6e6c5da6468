// Key preprocess of one batch after the sort: unique keys, run starts, inverse index, owner buckets,
// resident offsets; and the push plan of the previous batch.
// Reference: csrc/core/preprocess.cu:11-182 (kernels generate_sort_kv, write_sort_result,
// preprocess_batch_data, compute_idx_map, block_cvt_offset_to_shape, decide_update and the
// cub RunLengthEncode / ExclusiveSum calls between them).
#include "kernels.h"
#include "radix_sort.h"
#include "run_lists.h"
#include "tile_sort.h"

namespace hctr {
namespace {

constexpr int kBlock = 256;
constexpr int kItems = 8;
constexpr int kTile = kBlock * kItems; // 2048: scan_blocks(n) sizes the scratch

// ids -> sort keys (owner << id_bits | id; they are the batch's copy of the ids as well), the range check, the reset
// of the batch's run counters, and the per-tile counts of the first sort pass' digit: a block works on one sort tile, so the sort
// needs no counting launch of its own for that pass.  This is the one kernel that reads the caller's buffer: the
// call may return when it is through.
template <typename K, int ITEMS>
__global__ __launch_bounds__(kSortBlock) void make_keys(const index_t *__restrict__ keys, uint32_t n, uint64_t id_max,
                                                         int id_bits, int nrank, const worker_t *__restrict__ root,
                                                         K *__restrict__ comp, uint32_t *__restrict__ err,
                                                         uint32_t *__restrict__ nlong, int dbits,
                                                         uint32_t *__restrict__ counts, bool ids32) {
  __shared__ uint32_t h[kSortMaxBins];
  const uint32_t nb = 1u << dbits, mask = nb - 1;
  if (counts)
    for (uint32_t i = threadIdx.x; i < nb; i += kSortBlock) h[i] = 0;
  if (blockIdx.x == 0 && threadIdx.x < kRunCounters && nlong) nlong[threadIdx.x] = 0; // counters of this batch
  const uint32_t base = blockIdx.x * (ITEMS * kSortBlock);
  uint64_t id[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = base + k * kSortBlock + threadIdx.x;
    // the caller's ids are read here and nowhere else (ids32: as narrowed on their way from pageable host memory)
    id[k] = i >= n ? 0 : ids32 ? (uint64_t)load_once(&((const uint32_t *)keys)[i]) : (uint64_t)load_once(&keys[i]);
  }
  __syncthreads();
  bool bad = false;
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = base + k * kSortBlock + threadIdx.x;
    if (i < n && id[k] >= id_max) { // also catches negative ids
      bad = true;
      id[k] = 0;
    }
  }
  if (bad) atomicOr(err, 1u);
  uint64_t owner[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) owner[k] = nrank > 1 ? root[id[k]] : 0;
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t i = base + k * kSortBlock + threadIdx.x;
    const K c = (K)((owner[k] << id_bits) | id[k]);
    if (i < n) comp[i] = c;
    if (counts) count_digit(h, (uint32_t)c & mask, i < n);
  }
  if (!counts) return; // the keys alone: another sort counts for itself
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < nb; i += kSortBlock) counts[(size_t)blockIdx.x * nb + i] = h[i];
}

// The unique pass works on tiles of kUTile sorted positions; position j of a tile is handled by thread (j % kUBlock)
// in round (j / kUBlock): every load and store below is coalesced across the wave.
#ifndef HCTR_UNIQUE_ITEMS
#define HCTR_UNIQUE_ITEMS 8
#endif
constexpr int kUBlock = 512, kUItems = HCTR_UNIQUE_ITEMS, kUTile = kUBlock * kUItems;
inline unsigned unique_tiles(uint32_t n) { return div_up(n, kUTile); }

// Heads (sorted positions that hold another key than the position before) are counted per chunk of sorted positions,
// in a form that needs no look at a neighbouring chunk: the heads of a chunk other than its first position, and the
// chunk's first and last key.  The last launch of the tile-sorted passes leaves these three per chunk (tile_sort.h);
// after the other sort head_count makes them, one chunk per tile of the unique pass.
template <typename K>
__global__ __launch_bounds__(kUBlock) void head_count(const K *__restrict__ sk, uint32_t n,
                                                      uint32_t *__restrict__ inner, K *__restrict__ first,
                                                      K *__restrict__ last) {
  __shared__ uint32_t sm[kUBlock / kWave + 1];
  const uint32_t base = blockIdx.x * kUTile;
  const unsigned lane = lane_id();
  K key[kUItems], edge[kUItems];
#pragma unroll
  for (int k = 0; k < kUItems; k++) {
    const uint32_t j = base + k * kUBlock + threadIdx.x;
    key[k] = j < n ? sk[j] : (K)0;
    edge[k] = (lane == 0 && j < n && j > base) ? sk[j - 1] : (K)0; // the key before a wave's first position
  }
  uint32_t c = 0;
#pragma unroll
  for (int k = 0; k < kUItems; k++) {
    const uint32_t j = base + k * kUBlock + threadIdx.x;
    const K up = (K)__shfl_up(key[k], 1, kWave);
    const K pk = lane == 0 ? edge[k] : up;
    c += (j < n) && j > base && key[k] != pk;
  }
  uint32_t total;
  block_exclusive_scan<kUBlock>(c, sm, total);
  if (threadIdx.x == 0) {
    inner[blockIdx.x] = total;
    first[blockIdx.x] = key[0];
    last[blockIdx.x] = sk[min(base + kUTile, n) - 1];
  }
}

// One block per tile of ITEMS * kUBlock sorted positions; position j of a tile is handled by thread (j % kUBlock) in
// round (j / kUBlock).  chunk: sorted positions per entry of the head counts (a divisor of the tile).
template <typename K, int ITEMS>
__global__ __launch_bounds__(kUBlock) void unique_emit(const K *__restrict__ sk, uint32_t n, int id_bits, int nrank,
                                                       const slot_t *__restrict__ slot,
                                                       const uint32_t *__restrict__ head_inner,
                                                       const K *__restrict__ head_first, const K *__restrict__ head_last,
                                                       uint32_t chunk, BatchView b, uint32_t *__restrict__ u_copy) {
  constexpr int NW = kUBlock / kWave;
  constexpr uint32_t kTileU = ITEMS * kUBlock;
  __shared__ uint32_t sm[NW + 1];
  __shared__ uint32_t wsum[ITEMS * NW + 1];
  const uint32_t base = blockIdx.x * kTileU;
  const unsigned lane = lane_id();
  const int w = threadIdx.x / kWave;
  // everything that comes from memory first: the keys of the tile, the key before every wave's first position and the
  // head counts of the chunks before the tile
  K key[ITEMS], edge[ITEMS], pk[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t j = base + k * kUBlock + threadIdx.x;
    key[k] = j < n ? sk[j] : (K)0;
    edge[k] = (lane == 0 && j < n && j > 0) ? sk[j - 1] : (K)0;
  }
  uint32_t s = 0;
  const uint32_t chunks_before = base / chunk;
  for (uint32_t i = threadIdx.x; i < chunks_before; i += kUBlock)
    s += head_inner[i] + ((i == 0 || head_first[i] != head_last[i - 1]) ? 1u : 0u);
  bool head[ITEMS];
  uint32_t before[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t j = base + k * kUBlock + threadIdx.x;
    const bool valid = j < n;
    const K up = (K)__shfl_up(key[k], 1, kWave);
    pk[k] = lane == 0 ? edge[k] : up;
    head[k] = valid && (j == 0 || key[k] != pk[k]);
    const uint64_t m = __ballot(head[k]);
    before[k] = __popcll(m & ((1ull << lane) - 1ull));
    if (lane == 0) wsum[k * NW + w] = __popcll(m);
  }
  // the directory lookups of the heads travel while the ranks are worked out
  const K id_mask = (K)(((uint64_t)1 << id_bits) - 1);
  slot_t off[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; k++) off[k] = head[k] ? slot[(uint64_t)(key[k] & id_mask)] : kNoSlot;
  uint32_t prefix;
  block_exclusive_scan<kUBlock>(s, sm, prefix); // unique ranks before this tile
  if (threadIdx.x < kWave) { // the wave totals, in item order, by one wave
    uint32_t run = 0;
    for (int i0 = 0; i0 < ITEMS * NW; i0 += kWave) {
      const bool in = i0 + (int)lane < ITEMS * NW;
      const uint32_t v = in ? wsum[i0 + lane] : 0u;
      const uint32_t inc = wave_inclusive_scan(v);
      if (in) wsum[i0 + lane] = run + inc - v;
      run += __shfl(inc, kWave - 1, kWave);
    }
  }
  __syncthreads();
  K *ukey = (K *)b.ukey;
#pragma unroll
  for (int k = 0; k < ITEMS; k++) {
    const uint32_t j = base + k * kUBlock + threadIdx.x;
    if (j >= n) continue;
    const uint32_t rank = prefix + wsum[k * NW + w] + before[k] + (head[k] ? 1u : 0u) - 1u;
    const int r = (int)(key[k] >> id_bits);
    if (head[k]) {
      ukey[rank] = key[k];
      b.run_start[rank] = j;
      b.uoff[rank] = off[k];
      const int r_prev = j == 0 ? -1 : (int)(pk[k] >> id_bits);
      for (int i = r_prev + 1; i <= r; i++) b.bucket_lo[i] = rank;
    }
    b.rank_sorted[j] = rank;
    if (j == n - 1) {
      const uint32_t U = rank + 1;
      *b.d_U = U;
      if (u_copy) *u_copy = U;
      b.run_start[U] = n;
      for (int i = r + 1; i <= nrank; i++) b.bucket_lo[i] = U;
    }
  }
}

// The inverse index in batch order (the reference's d_idx_map).  The hot path works in sorted order
// (sorted_arg + rank_sorted are the same mapping, grouped by key) and never reads this array; it is
// materialised on request.
__global__ __launch_bounds__(kBlock) void scatter_idx_map(BatchView b) {
  const uint32_t j = blockIdx.x * kBlock + threadIdx.x;
  if (j < b.n) b.idx_map[b.sorted_arg[j]] = b.rank_sorted[j];
}

// the run lists of a batch by a launch of their own (run_lists.h), for a batch no gather builds them for
__global__ __launch_bounds__(kRunListBlock) void list_long_runs(BatchView b) {
  __shared__ uint32_t cnt[kRunLists], base[kRunLists];
  list_runs_chunk(b, blockIdx.x, cnt, base);
}

// ---- generic device-wide exclusive scan (two launches, no inter-block waiting) ----------------------
__global__ __launch_bounds__(kBlock) void scan_block_sums(const uint32_t *__restrict__ in, uint32_t n_max,
                                                          const uint32_t *__restrict__ d_n,
                                                          uint32_t *__restrict__ block_sums) {
  __shared__ uint32_t sm[kBlock / kWave + 1];
  const uint32_t n = d_n ? min(*d_n, n_max) : n_max;
  const uint32_t j0 = blockIdx.x * kTile + threadIdx.x * kItems;
  uint32_t c = 0;
#pragma unroll
  for (int k = 0; k < kItems; k++) c += (j0 + k < n) ? in[j0 + k] : 0u;
  uint32_t total;
  block_exclusive_scan<kBlock>(c, sm, total);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}

__global__ __launch_bounds__(kBlock) void scan_emit(const uint32_t *__restrict__ in, uint32_t *__restrict__ out,
                                                    uint32_t n_max, const uint32_t *__restrict__ d_n,
                                                    const uint32_t *__restrict__ block_sums,
                                                    uint32_t *__restrict__ total_out) {
  __shared__ uint32_t sm[kBlock / kWave + 1];
  const uint32_t n = d_n ? min(*d_n, n_max) : n_max;
  uint32_t s = 0;
  for (uint32_t i = threadIdx.x; i < blockIdx.x; i += kBlock) s += block_sums[i];
  uint32_t prefix;
  block_exclusive_scan<kBlock>(s, sm, prefix);
  const uint32_t j0 = blockIdx.x * kTile + threadIdx.x * kItems;
  uint32_t v[kItems], c = 0;
#pragma unroll
  for (int k = 0; k < kItems; k++) {
    v[k] = (j0 + k < n) ? in[j0 + k] : 0u;
    c += v[k];
  }
  uint32_t total;
  uint32_t run = prefix + block_exclusive_scan<kBlock>(c, sm, total);
#pragma unroll
  for (int k = 0; k < kItems; k++) {
    if (j0 + k < n) out[j0 + k] = run;
    run += v[k];
  }
  if (total_out && blockIdx.x == gridDim.x - 1 && threadIdx.x == kBlock - 1) *total_out = run;
}

template <typename K>
__global__ __launch_bounds__(kBlock) void decide_update(TableView t, int id_bits, BatchView p,
                                                        uint32_t *__restrict__ need) {
  const uint32_t u = blockIdx.x * kBlock + threadIdx.x;
  if (u >= *p.d_U) return;
  const K key = ((const K *)p.ukey)[u];
  const int r = (int)(key >> id_bits);
  const slot_t o = p.uoff[u];
  const version_t cnt = (version_t)(p.run_start[u + 1] - p.run_start[u]);
  uint32_t nd;
  if (r == t.rank) nd = 0;
  else if (o == kNoSlot) nd = 1;
  else nd = (t.upd[o] + cnt <= t.push_bound) ? 0 : 1;
  need[u] = nd;
}

__global__ void bucket_counts(BatchView b, const uint32_t *__restrict__ prefix, const uint32_t *__restrict__ total,
                              int nrank, uint64_t *__restrict__ cnt_out, uint64_t *__restrict__ host_out) {
  const int d = threadIdx.x;
  if (d > nrank) return;
  uint64_t c = 0;
  if (d < nrank) {
    const uint32_t U = *b.d_U;
    const uint32_t lo = b.bucket_lo[d], hi = b.bucket_lo[d + 1];
    const uint32_t a = lo >= U ? *total : prefix[lo];
    const uint32_t e = hi >= U ? *total : prefix[hi];
    c = U ? (uint64_t)(e - a) : 0;
  }
  cnt_out[d] = c;
  host_out[d] = c; // pinned host memory: the caller sizes the push buffers from it, no copy in between
}

__global__ void bucket_sizes(BatchView b, int nrank, uint64_t *__restrict__ cnt_out, uint64_t *__restrict__ host_out,
                             uint32_t *__restrict__ host_U) {
  const int d = threadIdx.x;
  if (d > nrank) return;
  const uint64_t c = d == nrank ? 0 : (uint64_t)(b.bucket_lo[d + 1] - b.bucket_lo[d]);
  cnt_out[d] = c;
  host_out[d] = c; // pinned host memory, like the number of unique keys beside it
  if (d == 0) *host_U = *b.d_U;
}

} // namespace

void launch_make_keys(hipStream_t s, const TableView &t, const KeyLayout &kl, const index_t *keys, uint32_t n,
                      void *comp_keys, uint32_t *err, uint32_t *nlong, uint32_t *sort_counts, bool ids32) {
  HCTR_CHECK(!ids32 || t.id_max <= 0xffffffffull, "internal: narrowed ids and a table of 2^32 rows or more");
  if (!n) return;
  const unsigned nblocks = (unsigned)sort_tiles(n);
  const int dbits = sort_first_digit_bits(kl.total_bits);
#define CALL(I)                                                                                                       \
  do {                                                                                                                \
    if (kl.wide)                                                                                                      \
      hipLaunchKernelGGL((make_keys<uint64_t, I>), dim3(nblocks), dim3(kSortBlock), 0, s, keys, n, t.id_max,          \
                         kl.id_bits, t.nrank, t.root, (uint64_t *)comp_keys, err, nlong, dbits, sort_counts,  \
                         ids32);         \
    else                                                                                                              \
      hipLaunchKernelGGL((make_keys<uint32_t, I>), dim3(nblocks), dim3(kSortBlock), 0, s, keys, n, t.id_max,          \
                         kl.id_bits, t.nrank, t.root, (uint32_t *)comp_keys, err, nlong, dbits, sort_counts,  \
                         ids32);         \
  } while (0)
  HCTR_SORT_ITEMS_DISPATCH(n, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_unique(hipStream_t s, const TableView &t, const KeyLayout &kl, const void *sorted_keys,
                   const BatchView &b, const HeadChunks &heads, bool count_heads, uint32_t *u_copy) {
  if (!b.n) return;
  // the tile of the pass: that of the sort that left the head counts, or kUTile when they are counted here
  const int items = count_heads ? kUItems : (int)(heads.chunk / kWave);
  const uint32_t chunk = count_heads ? (uint32_t)kUTile : heads.chunk;
  const unsigned nb = div_up(b.n, (size_t)items * kUBlock);
#define EMIT(K, I)                                                                                                  \
  hipLaunchKernelGGL((unique_emit<K, I>), dim3(nb), dim3(kUBlock), 0, s, (const K *)sorted_keys, b.n, kl.id_bits,   \
                     t.nrank, t.slot, heads.inner, (const K *)heads.first, (const K *)heads.last, chunk, b, u_copy)
#define EMIT_K(K)                                                                                          \
  do {                                                                                                     \
    if (count_heads)                                                                                       \
      hipLaunchKernelGGL(head_count<K>, dim3(nb), dim3(kUBlock), 0, s, (const K *)sorted_keys, b.n, heads.inner, \
                         (K *)heads.first, (K *)heads.last);                                              \
    switch (items) {                                                                                       \
      case 2: EMIT(K, 2); break;                                                                           \
      case 4: EMIT(K, 4); break;                                                                           \
      case 8: EMIT(K, 8); break;                                                                           \
      case 13: EMIT(K, 13); break;                                                                         \
      case 16: EMIT(K, 16); break;                                                                         \
      default: throw Error("hetuCTR: internal: no unique pass for this tile shape");                       \
    }                                                                                                      \
  } while (0)
  if (kl.wide) EMIT_K(uint64_t);
  else EMIT_K(uint32_t);
#undef EMIT_K
#undef EMIT
  HCTR_HIP(hipGetLastError());
}

void launch_idx_map(hipStream_t s, const BatchView &b) {
  if (!b.n) return;
  hipLaunchKernelGGL(scatter_idx_map, dim3(div_up(b.n, kBlock)), dim3(kBlock), 0, s, b);
  HCTR_HIP(hipGetLastError());
}

void launch_list_long_runs(hipStream_t s, const BatchView &b) { // the class counters were zeroed by make_keys
  if (!b.n) return;
  hipLaunchKernelGGL(list_long_runs, dim3(div_up(b.n, kRunListBlock)), dim3(kRunListBlock), 0, s, b);
  HCTR_HIP(hipGetLastError());
}

void launch_exclusive_scan(hipStream_t s, const uint32_t *in, uint32_t *out, uint32_t n_max, const uint32_t *d_n,
                           uint32_t *block_sums, uint32_t *total) {
  if (!n_max) {
    if (total) HCTR_HIP(hipMemsetAsync(total, 0, sizeof(uint32_t), s));
    return;
  }
  const unsigned nb = div_up(n_max, kTile);
  hipLaunchKernelGGL(scan_block_sums, dim3(nb), dim3(kBlock), 0, s, in, n_max, d_n, block_sums);
  hipLaunchKernelGGL(scan_emit, dim3(nb), dim3(kBlock), 0, s, in, out, n_max, d_n, block_sums, total);
  HCTR_HIP(hipGetLastError());
}

void launch_decide_update(hipStream_t s, const TableView &t, const KeyLayout &kl, const BatchView &prev,
                          uint32_t *need) {
  if (!prev.n) return;
  if (kl.wide)
    hipLaunchKernelGGL(decide_update<uint64_t>, dim3(div_up(prev.n, kBlock)), dim3(kBlock), 0, s, t, kl.id_bits, prev, need);
  else
    hipLaunchKernelGGL(decide_update<uint32_t>, dim3(div_up(prev.n, kBlock)), dim3(kBlock), 0, s, t, kl.id_bits, prev, need);
  HCTR_HIP(hipGetLastError());
}

void launch_bucket_counts(hipStream_t s, const BatchView &b, const uint32_t *prefix, const uint32_t *total,
                          int nrank, uint64_t *cnt_out, uint64_t *host_out) {
  hipLaunchKernelGGL(bucket_counts, dim3(1), dim3(nrank + 1), 0, s, b, prefix, total, nrank, cnt_out, host_out);
  HCTR_HIP(hipGetLastError());
}

void launch_bucket_sizes(hipStream_t s, const BatchView &b, int nrank, uint64_t *cnt_out, uint64_t *host_out,
                         uint32_t *host_U) {
  hipLaunchKernelGGL(bucket_sizes, dim3(1), dim3(nrank + 1), 0, s, b, nrank, cnt_out, host_out, host_U);
  HCTR_HIP(hipGetLastError());
}

} // namespace hctr
