// Pull side and owner side of a step: version lookup for the query, applying pushed rows, deciding which
// queried rows are outdated, packing the rows to return, refreshing cached rows and the final gather of
// every key's row into the caller's output.
// Reference: csrc/core/generate_query.cu:91-106, csrc/core/handle_query.cu:7-116,
// csrc/core/writeback.cu:8-56.
#include "kernels.h"
#include "run_lists.h"

namespace hctr {
namespace {

constexpr int kBlock = 256;
static_assert(kBlock == kRunListBlock, "the gather's blocks list runs chunk by chunk");
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int VEC> struct RowVec;
template <> struct RowVec<4> { typedef floatx4 T; };
template <> struct RowVec<1> { typedef float T; };

// The queries of a step (csrc/core/generate_query.cu:91-106): per unique key its id and the version of the local copy
// (invalid if the key is not resident here), written where the key's owner reads its queries: place u + delta[owner]
// of a receive area all owners share.
template <typename K>
__global__ __launch_bounds__(kBlock) void build_queries(TableView t, int id_bits, BatchView c,
                                                        const uint32_t *__restrict__ delta, index_t *__restrict__ q_idx,
                                                        version_t *__restrict__ q_ver) {
  const uint32_t u = blockIdx.x * kBlock + threadIdx.x;
  if (u >= *c.d_U) return;
  const slot_t o = c.uoff[u];
  const K key = ((const K *)c.ukey)[u];
  const uint32_t pos = u + delta[(uint32_t)(key >> id_bits)];
  q_idx[pos] = (index_t)(key & (K)(((uint64_t)1 << id_bits) - 1));
  q_ver[pos] = o != kNoSlot ? t.ver[o] : kInvalidVersion;
}

// ---- owner side: every kernel below serves ALL shards of a loopback group in one launch (blockIdx.y = shard), the
// way the shards' GPUs would work side by side; with one shard per process the grid is one row high.
//
// Received pushes (csrc/core/handle_query.cu:106-116 applies them source by source, in rank order).  The rows that hit
// one target must be added in source order, so a target's rows all go to one block: every source's segment of the
// receive buffer is ascending in id (it is a slice of the sender's sorted unique keys), block b takes the ids
// between two splitters drawn from the longest segment, finds that id range in every other segment by binary search,
// and walks the sources in order with a barrier between them.  Inside a source ids are distinct, so its rows are
// applied in parallel, kAhead rows per group of LPR lanes at a time.
__device__ __forceinline__ uint32_t lower_bound_id(const index_t *__restrict__ a, uint32_t lo, uint32_t hi, index_t x) {
  while (lo < hi) { // first position in [lo, hi) whose id is >= x
    const uint32_t mid = lo + (hi - lo) / 2;
    if (a[mid] < x) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}
#ifndef HCTR_APPLY_AHEAD
#define HCTR_APPLY_AHEAD 2
#endif
#ifndef HCTR_APPLY_BATCHES
#define HCTR_APPLY_BATCHES 1
#endif
// Rows of one source a group works on together (distinct ids, hence distinct targets), and batches of that many rows
// per group and block.  Small blocks measured fastest: the kernel is a stream of independent read-modify-writes, and
// what limits it is how evenly the blocks spread over the chip, not the loads one wave keeps in flight.
constexpr int kApplyAhead = HCTR_APPLY_AHEAD;
constexpr int kApplyBatches = HCTR_APPLY_BATCHES;
// The slot of an id the shard owns, kNoSlot for any other id.  Slots below n_cached hold the cached copies of rows
// other shards own, so the slot alone tells (no look at the owner table).
__device__ __forceinline__ slot_t owned_slot(const slot_t *__restrict__ slot, uint64_t id, uint64_t id_max, uint32_t n_cached) {
  if (id >= id_max) return kNoSlot;
  const slot_t o = slot[id];
  return (o != kNoSlot && (uint32_t)o >= n_cached) ? o : kNoSlot;
}
template <int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void apply_remote_all(const OwnerShard *__restrict__ shards, int nsrc,
                                                           uint32_t rows_per_block) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const OwnerShard &S = shards[blockIdx.y];
  if (blockIdx.x >= S.push_blocks) return;
  const index_t *__restrict__ rg_idx = S.rg_idx;
  const version_t *__restrict__ rg_cnt = S.rg_cnt;
  const embed_t *__restrict__ rg_val = S.rg_val;
  const slot_t *__restrict__ slot = S.t.slot;
  embed_t *__restrict__ emb = S.t.emb;
  version_t *__restrict__ ver = S.t.ver;
  const uint64_t id_max = S.t.id_max;
  const uint32_t n_cached = S.t.n_cached, W = S.t.width;
  __shared__ uint32_t lo[256], hi[256];
  const int longest = S.longest;
  const uint32_t big_lo = S.rg_seg[longest], big_hi = S.rg_seg[longest + 1];
  const uint32_t first = big_lo + blockIdx.x * rows_per_block, last = first + rows_per_block;
  for (int s = threadIdx.x; s < nsrc; s += kBlock) {
    const uint32_t a = S.rg_seg[s], b = S.rg_seg[s + 1];
    if (s == longest) { // the splitters are this segment's own rows
      lo[s] = first;
      hi[s] = min(last, big_hi);
    } else if (a == b) {
      lo[s] = hi[s] = a;
    } else {
      // block 0 starts below every id, the last block ends above every id
      lo[s] = blockIdx.x == 0 ? a : lower_bound_id(rg_idx, a, b, rg_idx[first]);
      hi[s] = last >= big_hi ? b : lower_bound_id(rg_idx, lo[s], b, rg_idx[last]);
    }
  }
  __syncthreads();
  const uint32_t gl = threadIdx.x % LPR;
  constexpr int kAhead = kApplyAhead;
  bool bad = false;
  for (int s = 0; s < nsrc; s++) {
    const uint32_t end = hi[s];
    for (uint32_t k0 = lo[s] + threadIdx.x / LPR; k0 < end; k0 += kGroups * kAhead) {
      slot_t o[kAhead];
      uint64_t id[kAhead];
#pragma unroll
      for (int a = 0; a < kAhead; a++) id[a] = (uint64_t)rg_idx[min(k0 + a * kGroups, end - 1)];
#pragma unroll
      for (int a = 0; a < kAhead; a++) {
        o[a] = owned_slot(slot, id[a], id_max, n_cached);
        if (k0 + a * kGroups >= end) o[a] = kNoSlot;
        else if (o[a] == kNoSlot) bad = true;
      }
      if (gl == 0) {
#pragma unroll
        for (int a = 0; a < kAhead; a++)
          if (o[a] != kNoSlot) ver[o[a]] += load_once(rg_cnt + k0 + a * kGroups);
      }
      for (uint32_t col = gl * VEC; col < W; col += LPR * VEC) {
        V cur[kAhead], add[kAhead];
#pragma unroll
        for (int a = 0; a < kAhead; a++) {
          if (o[a] == kNoSlot) continue;
          cur[a] = *(const V *)(emb + (size_t)o[a] * W + col);
          add[a] = load_once((const V *)(rg_val + (size_t)(k0 + a * kGroups) * W + col)); // read once: keep it out of the caches
        }
#pragma unroll
        for (int a = 0; a < kAhead; a++)
          if (o[a] != kNoSlot) *(V *)(emb + (size_t)o[a] * W + col) = cur[a] + add[a];
      }
    }
    __syncthreads(); // the next source may push to the same rows
  }
  if (bad && gl == 0) atomicOr(S.err, 2u);
}

// Owner side of the pull (csrc/core/handle_query.cu:7-78) in three launches; the first two work on tiles of kBlock
// received queries, one query per thread.
// decide_count: the outdated flag of every query (pull rule, self-exempt, :47-54) and the number of flags per tile.
// scan_positions: a tile's flags scanned behind the tiles before it -> position of every flagged query among the
// returned rows (:56-57, :74-75), and the first returned row of every requester's segment (:59-61) written both to
// device memory, where place_returns reads it, and to the host.
// pack_rows: version and row of every flagged query packed at its position (:24-40), from the list of their slots
// that scan_positions leaves.
// One block.  Thread d, owner: its queries per requester in rank order (rq_seg), their number, the tiles of its flag
// scan; then the owners' pieces of the area in rank order; thread s, requester: what it adds to a unique key's rank
// per owner (query_delta), and what owner d adds to the place of one of s' queries to get the place of its flag in
// s' array (got_delta: s' flags stand in owner order).  Up to kPlaceLds shards the matrix of counts is fetched into LDS
// by all threads at once (one memory round trip instead of one per entry and thread).
constexpr int kPlaceLds = 48;
struct PlaceSources { // of the first kPlaceLds shards: where their counts lie, and whether they ask at all
  const uint64_t *send_cnt[kPlaceLds];
  uint32_t n_keys[kPlaceLds];
};
__global__ __launch_bounds__(kBlock) void place_queries(OwnerShard *shards, int R, QueryArea area, PlaceSources src) {
  __shared__ uint32_t sm[kBlock / kWave + 1];
  __shared__ uint32_t base[kBlock];
  __shared__ uint32_t cnt[kPlaceLds * kPlaceLds];  // [requester][owner] unique keys asked for
  __shared__ uint32_t segm[kPlaceLds * kPlaceLds]; // [owner][requester] first query of the requester at the owner
  const int t = threadIdx.x;
  const bool in_lds = R <= kPlaceLds;
  if (in_lds) {
    for (int i = t; i < R * R; i += kBlock) {
      const int s = i / R, d = i % R;
      cnt[i] = src.n_keys[s] ? (uint32_t)src.send_cnt[s][d] : 0u;
    }
    __syncthreads();
  }
  auto asked = [&](int s, int d) -> uint32_t { // unique keys requester s asks owner d for
    if (in_lds) return cnt[s * R + d];
    return shards[s].n_keys ? (uint32_t)shards[s].send_cnt[d] : 0u;
  };
  uint32_t Q = 0;
  if (t < R) {
    OwnerShard &D = shards[t];
    for (int s = 0; s < R; s++) {
      D.rq_seg[s] = Q;
      if (in_lds) segm[t * R + s] = Q;
      Q += asked(s, t);
    }
    D.rq_seg[R] = Q;
    D.q = Q;
    D.query_tiles = max(1u, (Q + kBlock - 1) / kBlock); // one tile even without queries: the segment table is written
  }
  uint32_t total;
  const uint32_t lo = block_exclusive_scan<kBlock>(Q, sm, total);
  base[t] = lo;
  if (t < R) {
    OwnerShard &D = shards[t];
    D.rq_idx = area.idx + lo;
    D.rq_ver = area.ver + lo;
    D.outdated = area.outdated + lo;
    D.q_slot = area.q_slot + lo;
    D.ret_slot = area.ret_slot + lo;
  }
  __syncthreads(); // rq_seg of every owner is written (global memory, this block), base[] too
  if (t < R) {
    uint32_t ulo = 0; // unique keys of requester t that belong to the owners before d
    for (int d = 0; d < R; d++) {
      const uint32_t seg = in_lds ? segm[d * R + t] : shards[d].rq_seg[t];
      // (place in the area) - (rank among the requester's unique keys), modulo 2^32 like the sum the kernel forms
      area.query_delta[(size_t)t * R + d] = base[d] + seg - ulo;
      shards[d].got_delta[t] = ulo - seg;
      ulo += asked(t, d);
    }
  }
}

__global__ __launch_bounds__(kBlock) void decide_count(const OwnerShard *__restrict__ shards, int nseg) {
  const OwnerShard &S = shards[blockIdx.y];
  if (blockIdx.x >= S.query_tiles) return;
  const TableView &t = S.t;
  __shared__ uint32_t wcnt[kBlock / kWave];
  __shared__ uint32_t sseg[258];
  for (int i = threadIdx.x; i <= nseg; i += kBlock) sseg[i] = S.rq_seg[i];
  __syncthreads();
  // the grid is cut from a guess (the number of queries is known on the device only): a block takes every gridDim.x-th tile
  for (uint32_t tile = blockIdx.x; tile < S.query_tiles; tile += gridDim.x) {
    const uint32_t k = tile * kBlock + threadIdx.x;
    uint32_t flag = 0;
    if (k < S.q) {
      const slot_t o = owned_slot(t.slot, (uint64_t)S.rq_idx[k], t.id_max, t.n_cached);
      S.q_slot[k] = o;
      // the requester: the segment of the receive buffer the query lies in (segments may be empty)
      uint32_t lo = 0, hi = nseg - 1;
      while (lo < hi) { // the first segment that ends behind k
        const uint32_t mid = (lo + hi) / 2;
        if (sseg[mid + 1] <= k) lo = mid + 1;
        else hi = mid;
      }
      if (o == kNoSlot) {
        atomicOr(S.err, 4u);
      } else {
        const version_t local = S.rq_ver[k], global = t.ver[o];
        const bool from_self = lo == (uint32_t)t.rank;
        const bool out = local == kInvalidVersion || local + t.pull_bound < global;
        flag = (out && !from_self) ? 1u : 0u;
      }
      S.outdated[k] = flag;
      shards[lo].got[k + S.got_delta[lo]] = flag; // the requester reads it from its own array
    }
    const uint64_t m = __ballot(flag != 0);
    if (lane_id() == 0) wcnt[threadIdx.x / kWave] = __popcll(m);
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t c = 0;
      for (int i = 0; i < kBlock / kWave; i++) c += wcnt[i];
      S.tile_cnt[tile] = c;
    }
    __syncthreads(); // wcnt is rewritten for the next tile
  }
}

__global__ __launch_bounds__(kBlock) void scan_positions(const OwnerShard *__restrict__ shards, int nseg) {
  const OwnerShard &S = shards[blockIdx.y];
  __shared__ uint32_t sm[kBlock / kWave + 1];
  __shared__ uint32_t excl[kBlock + 1]; // position of every query of the tile among the returned rows; [kBlock]: after it
  const uint32_t q = S.q;
  for (uint32_t tile = blockIdx.x; tile < S.query_tiles; tile += gridDim.x) { // as in decide_count
    const uint32_t tile_lo = tile * kBlock, k = tile_lo + threadIdx.x;
    const uint32_t f = k < q ? S.outdated[k] : 0u;
    uint32_t s = 0;
    for (uint32_t i = threadIdx.x; i < tile; i += kBlock) s += S.tile_cnt[i];
    uint32_t before;
    block_exclusive_scan<kBlock>(s, sm, before); // flagged queries in the tiles before this one
    uint32_t total;
    const uint32_t pos = before + block_exclusive_scan<kBlock>(f, sm, total);
    if (f) S.ret_slot[pos] = S.q_slot[k]; // the rows to return, in the order they go back
    excl[threadIdx.x] = pos;
    if (threadIdx.x == 0) excl[kBlock] = before + total;
    __syncthreads();
    // the first returned row of a requester's segment is the position of the segment's first query
    const bool last_tile = tile == S.query_tiles - 1;
    for (int g = threadIdx.x; g <= nseg; g += kBlock) {
      const uint32_t start = S.rq_seg[g];
      uint32_t v = ~0u;
      if (start >= tile_lo && start < tile_lo + kBlock && start < q) v = excl[start - tile_lo];
      else if (last_tile && start >= q) v = excl[kBlock]; // segments that start at the end: the total
      if (v != ~0u) {
        S.seg_dev[g] = v;
        S.seg_host[g] = v;
      }
    }
    if (last_tile && threadIdx.x == 0) S.seg_host[257] = *S.err;
    __syncthreads(); // excl is rewritten for the next tile
  }
}

// Where the rows an owner returns stand in the requesters' buffers: a requester's rows arrive in owner order
// (csrc/core/all2all.cu:89-130), and how many rows an owner returns to a requester is only known on the device.
// Thread (owner d, requester s): ret_delta of d for s = rows the owners before d return to s, minus the start of s'
// segment in d's own return order.
__global__ void place_returns(const OwnerShard *__restrict__ shards, int nrank) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (uint32_t)nrank * nrank) return;
  const int d = i / nrank, s = i % nrank;
  uint32_t before = 0;
  for (int e = 0; e < d; e++) before += shards[e].seg_dev[s + 1] - shards[e].seg_dev[s];
  shards[d].ret_delta[s] = before - shards[d].seg_dev[s];
}

// kPackAhead rows to return per group of LPR lanes; which rows, scan_positions has listed.  A row goes straight into
// the buffers of the shard that asked for it (in one process a plain device address, between GPUs peer memory).
#ifndef HCTR_PACK_AHEAD
#define HCTR_PACK_AHEAD 2
#endif
constexpr int kPackAhead = HCTR_PACK_AHEAD;
template <int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void pack_rows(const OwnerShard *__restrict__ shards, int nseg) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  __shared__ uint32_t sseg[258], sdelta[257];
  const OwnerShard &S = shards[blockIdx.y];
  for (int i = threadIdx.x; i <= nseg; i += kBlock) sseg[i] = S.seg_dev[i];
  for (int i = threadIdx.x; i < nseg; i += kBlock) sdelta[i] = S.ret_delta[i];
  __syncthreads();
  const uint32_t total = sseg[nseg]; // rows this shard returns: known on the device only, the grid is cut for the most
  const embed_t *__restrict__ emb = S.t.emb;
  const uint32_t gl = threadIdx.x % LPR, W = S.t.width;
  for (uint32_t k0 = blockIdx.x * (kGroups * kPackAhead) + threadIdx.x / LPR; k0 < total; k0 += gridDim.x * (kGroups * kPackAhead)) {
  slot_t o[kPackAhead];
#pragma unroll
  for (int a = 0; a < kPackAhead; a++) o[a] = k0 + a * kGroups < total ? S.ret_slot[k0 + a * kGroups] : kNoSlot;
  // the requester of every row: the segment of the return order it lies in (segments may be empty)
  embed_t *dst_val[kPackAhead];
  version_t *dst_ver[kPackAhead];
#pragma unroll
  for (int a = 0; a < kPackAhead; a++) {
    const uint32_t k = min(k0 + a * kGroups, total - 1);
    uint32_t lo = 0, hi = nseg - 1;
    while (lo < hi) { // the first segment that ends behind k
      const uint32_t mid = (lo + hi) / 2;
      if (sseg[mid + 1] <= k) lo = mid + 1;
      else hi = mid;
    }
    const uint32_t row = k + sdelta[lo];
    dst_val[a] = shards[lo].in_val + (size_t)row * W;
    dst_ver[a] = shards[lo].in_ver + row;
  }
  if (gl == 0) {
#pragma unroll
    for (int a = 0; a < kPackAhead; a++)
      if (o[a] != kNoSlot) *dst_ver[a] = S.t.ver[o[a]];
  }
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC) {
    V v[kPackAhead];
#pragma unroll
    for (int a = 0; a < kPackAhead; a++)
      if (o[a] != kNoSlot) v[a] = *(const V *)(emb + (size_t)o[a] * W + col);
#pragma unroll
    for (int a = 0; a < kPackAhead; a++)
      if (o[a] != kNoSlot) __builtin_nontemporal_store(v[a], (V *)(dst_val[a] + col)); // read next by another shard's kernels
  }
  }
}

// What comes back per unique key of the step, in two launches over tiles of kRTile keys:
//  got_tile_sums   returned rows per tile
//  remote_emit     ret_i[u] = index of u's row among the returned rows (exclusive scan of the flags; a tile adds up the
//                  sums of the tiles before it itself); src_row[u] = where the gather finds the row: the resident offset,
//                  or (top bit set) that index; and the counts of the step: [0] cached and fresh enough, [1] not stored
//                  here, [2] cached and refreshed, [3] bit 3: an owned row came back as outdated (it never may).
// Atomics on one address are served one after the other, so every thread counts its keys in registers and a block
// adds its totals once.  The block that finishes last hands the totals to the host (pinned memory) and puts the device
// counters back to zero for the next step: no clearing launch before, no copy after.
constexpr uint32_t kReturnedRow = 0x80000000u;
constexpr int kRItems = 8, kRTile = kBlock * kRItems; // 2048 keys: the tile scan_blocks() sizes the scratch for
__global__ __launch_bounds__(kBlock) void got_tile_sums(const uint32_t *__restrict__ got, const uint32_t *__restrict__ d_U,
                                                        uint32_t *__restrict__ tile_sums) {
  __shared__ uint32_t sm[kBlock / kWave + 1];
  const uint32_t U = *d_U; // the grid is cut for the batch's keys: the host has not seen the number of unique ones
  if (blockIdx.x * kRTile >= U) return;
  const uint32_t j0 = blockIdx.x * kRTile + threadIdx.x * kRItems;
  uint32_t c = 0;
#pragma unroll
  for (int k = 0; k < kRItems; k++) c += (j0 + k < U) ? got[j0 + k] : 0u;
  uint32_t total;
  block_exclusive_scan<kBlock>(c, sm, total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}
__global__ __launch_bounds__(kBlock) void remote_emit(TableView t, BatchView c, const uint32_t *__restrict__ got,
                                                      const uint32_t *__restrict__ tile_sums,
                                                      uint32_t *__restrict__ ret_i, uint32_t *__restrict__ src_row,
                                                      uint32_t *__restrict__ stats, uint32_t *__restrict__ host_stats) {
  __shared__ uint32_t sm[kBlock / kWave + 1];
  const uint32_t U = *c.d_U;
  const uint32_t tiles = (U + kRTile - 1) / kRTile; // of the grid's blocks (cut for the batch's keys) these have work
  if (blockIdx.x >= tiles) return;
  __shared__ uint32_t tot[4];
  __shared__ bool last;
  if (threadIdx.x < 4) tot[threadIdx.x] = 0;
  uint32_t s = 0;
  for (uint32_t i = threadIdx.x; i < blockIdx.x; i += kBlock) s += tile_sums[i];
  uint32_t prefix;
  block_exclusive_scan<kBlock>(s, sm, prefix); // its total: returned rows in the tiles before this one
  const uint32_t j0 = blockIdx.x * kRTile + threadIdx.x * kRItems;
  uint32_t g[kRItems], mine = 0;
  slot_t o[kRItems];
#pragma unroll
  for (int k = 0; k < kRItems; k++) {
    const bool in = j0 + k < U;
    g[k] = in ? got[j0 + k] : 0u;
    o[k] = in ? c.uoff[j0 + k] : 0;
    mine += g[k];
  }
  uint32_t total;
  uint32_t run = prefix + block_exclusive_scan<kBlock>(mine, sm, total);
  uint32_t n0 = 0, n1 = 0, n2 = 0, bad = 0;
#pragma unroll
  for (int k = 0; k < kRItems; k++) {
    if (j0 + k < U) {
      ret_i[j0 + k] = run;
      src_row[j0 + k] = o[k] == kNoSlot ? (kReturnedRow | run) : (uint32_t)o[k];
      if (o[k] == kNoSlot) n1++;
      else if ((uint32_t)o[k] < t.n_cached) {
        if (g[k]) n2++;
        else n0++;
      } else if (g[k]) {
        bad = 8u;
      }
    }
    run += g[k];
  }
  for (int d = 32; d; d >>= 1) {
    n0 += __shfl_down(n0, d);
    n1 += __shfl_down(n1, d);
    n2 += __shfl_down(n2, d);
    bad |= __shfl_down(bad, d);
  }
  if (threadIdx.x % 64 == 0) {
    atomicAdd(&tot[0], n0);
    atomicAdd(&tot[1], n1);
    atomicAdd(&tot[2], n2);
    atomicOr(&tot[3], bad);
  }
  __syncthreads();
  if (threadIdx.x < 3 && tot[threadIdx.x]) atomicAdd(&stats[threadIdx.x], tot[threadIdx.x]);
  if (threadIdx.x == 3 && tot[3]) atomicOr(&stats[3], tot[3]);
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence();
    last = atomicAdd(&stats[4], 1u) == tiles - 1;
  }
  __syncthreads();
  if (last && threadIdx.x < 4) {
    __threadfence();
    host_stats[threadIdx.x] = atomicExch(&stats[threadIdx.x], 0u);
    if (threadIdx.x == 0) stats[4] = 0;
  }
}

// one group per unique rank of the current batch
template <int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void refresh(TableView t, BatchView c, PullArgs a) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const uint32_t U = *c.d_U, gl = threadIdx.x % LPR, W = t.width;
  for (uint32_t u = blockIdx.x * kGroups + threadIdx.x / LPR; u < U; u += gridDim.x * kGroups) {
    const slot_t o = c.uoff[u];
    const bool got = a.got[u] != 0;
    if (!got || o == kNoSlot || (uint32_t)o >= t.n_cached) continue; // (an owned row that came back is reported by remote_emit)
    const uint32_t k = a.ret_i[u];
    if (gl == 0) t.ver[o] = a.in_ver[k];
    for (uint32_t col = gl * VEC; col < W; col += LPR * VEC)
      *(V *)(t.emb + (size_t)o * W + col) =
          *(const V *)(a.in_val + (size_t)k * W + col) + *(const V *)(t.pend + (size_t)o * W + col);
  }
}

// Gather in SORTED order: one group per kRows consecutive sorted positions.  Duplicates of a key are adjacent,
// so a table row is fetched from HBM once and re-read from cache for its other occurrences; every output row is
// written whole, once, with non-temporal stores, at the batch position sorted_arg names.
#ifndef HCTR_GATHER_ROWS
#define HCTR_GATHER_ROWS 8
#endif
constexpr int kRows = HCTR_GATHER_ROWS;
// kStream: dst is written with nontemporal stores (a compile-time choice: merged into one store by the compiler, a
// run-time one loses the hint)
template <int VEC, int LPR, bool kLocalOnly, bool kStream>
__global__ __launch_bounds__(kBlock) void gather(TableView t, BatchView c, PullArgs a) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const uint32_t n = c.n, W = t.width;
  if (blockIdx.x < a.list_chunks) { // the batch's run lists for its push one step later, before the block's own rows
    __shared__ uint32_t cnt[kRunLists], base[kRunLists];
    for (uint32_t chunk = blockIdx.x; chunk < a.list_chunks; chunk += gridDim.x) list_runs_chunk(c, chunk, cnt, base);
  }
  const uint32_t j0 = (blockIdx.x * kGroups + threadIdx.x / LPR) * kRows;
  if (j0 >= n) return;
  const uint32_t gl = threadIdx.x % LPR;
  const embed_t *src[kRows];
  embed_t *dst[kRows];
#pragma unroll
  for (int k = 0; k < kRows; k++) {
    const uint32_t j = min(j0 + k, n - 1);
    const uint32_t u = c.rank_sorted[j];
    const uint32_t i = c.sorted_arg[j];
    if (kLocalOnly) {
      src[k] = t.emb + (size_t)c.uoff[u] * W;
    } else {
      const uint32_t r = a.src_row[u];
      src[k] = (r & kReturnedRow) ? a.in_val + (size_t)(r & ~kReturnedRow) * W : t.emb + (size_t)r * W;
    }
    dst[k] = a.dst + (size_t)i * W;
  }
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC) {
    V v[kRows];
#pragma unroll
    for (int k = 0; k < kRows; k++) v[k] = *(const V *)(src[k] + col);
#pragma unroll
    for (int k = 0; k < kRows; k++)
      if (j0 + k < n) {
        if (kStream) __builtin_nontemporal_store(v[k], (V *)(dst[k] + col));
        else *(V *)(dst[k] + col) = v[k];
      }
  }
}

// Gather in BATCH order straight from the batch's keys, for one shard: dst[i] = emb[slot[id of position i]].  It needs
// nothing of the batch's index (sort, unique pass), so a step whose index is longer than its push -- a small batch --
// does not wait for it; what it gives up is the order in which the duplicates of a key are adjacent, which only matters
// once the rows of a batch no longer fit the caches.
template <int VEC, int LPR, typename K, bool kStream>
__global__ __launch_bounds__(kBlock) void gather_direct(TableView t, const K *__restrict__ keys, int id_bits, uint32_t n,
                                                        embed_t *__restrict__ dst_rows) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const uint32_t W = t.width;
  const uint32_t i0 = (blockIdx.x * kGroups + threadIdx.x / LPR) * kRows;
  if (i0 >= n) return;
  const uint32_t gl = threadIdx.x % LPR;
  const K id_mask = (K)(((uint64_t)1 << id_bits) - 1);
  const embed_t *src[kRows];
#pragma unroll
  for (int k = 0; k < kRows; k++) {
    const uint32_t i = min(i0 + k, n - 1);
    src[k] = t.emb + (size_t)t.slot[(uint64_t)(keys[i] & id_mask)] * W; // one shard: every id is resident
  }
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC) {
    V v[kRows];
#pragma unroll
    for (int k = 0; k < kRows; k++) v[k] = *(const V *)(src[k] + col);
#pragma unroll
    for (int k = 0; k < kRows; k++)
      if (i0 + k < n) {
        V *d = (V *)(dst_rows + (size_t)(i0 + k) * W + col);
        if (kStream) __builtin_nontemporal_store(v[k], d);
        else *d = v[k];
      }
  }
}

// Sum-pooled lookups: one group per bag of `bag` consecutive batch positions.  The rows of the bag are requested
// kPoolAhead at a time and added in position order (fp32, starting from the first row), so a bag costs one output
// row instead of `bag`.  Works in batch order, through the inverse index of the batch.
constexpr int kPoolAhead = 8;
template <int VEC, int LPR, bool kLocalOnly>
__global__ __launch_bounds__(kBlock) void gather_pooled(TableView t, BatchView c, PullArgs a, uint32_t bag,
                                                        uint32_t n_bags) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  if (blockIdx.x < a.list_chunks) { // the batch's run lists, as in gather
    __shared__ uint32_t cnt[kRunLists], base[kRunLists];
    for (uint32_t chunk = blockIdx.x; chunk < a.list_chunks; chunk += gridDim.x) list_runs_chunk(c, chunk, cnt, base);
  }
  const uint32_t b = blockIdx.x * kGroups + threadIdx.x / LPR;
  if (b >= n_bags) return;
  const uint32_t gl = threadIdx.x % LPR, W = t.width;
  const uint32_t i0 = b * bag;
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC) {
    V acc;
    for (uint32_t h0 = 0; h0 < bag; h0 += kPoolAhead) {
      const embed_t *src[kPoolAhead];
#pragma unroll
      for (int k = 0; k < kPoolAhead; k++) {
        const uint32_t u = c.idx_map[i0 + min(h0 + k, bag - 1)];
        if (kLocalOnly) {
          src[k] = t.emb + (size_t)c.uoff[u] * W;
        } else {
          const uint32_t r = a.src_row[u];
          src[k] = (r & kReturnedRow) ? a.in_val + (size_t)(r & ~kReturnedRow) * W : t.emb + (size_t)r * W;
        }
      }
      V v[kPoolAhead];
#pragma unroll
      for (int k = 0; k < kPoolAhead; k++) v[k] = *(const V *)(src[k] + col);
#pragma unroll
      for (int k = 0; k < kPoolAhead; k++) {
        if (h0 + k == 0) acc = v[k];
        else if (h0 + k < bag) acc = acc + v[k];
      }
    }
    __builtin_nontemporal_store(acc, (V *)(a.dst + (size_t)b * W + col));
  }
}

// The same for one shard from the batch's keys in batch order (as gather_direct): a bag's positions are consecutive in
// the batch, so this order costs no locality the other would have, and nothing of the batch's index is needed.
template <int VEC, int LPR, typename K>
__global__ __launch_bounds__(kBlock) void gather_pooled_direct(TableView t, const K *__restrict__ keys, int id_bits,
                                                               embed_t *__restrict__ dst_rows, uint32_t bag, uint32_t n_bags) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const uint32_t b = blockIdx.x * kGroups + threadIdx.x / LPR;
  if (b >= n_bags) return;
  const uint32_t gl = threadIdx.x % LPR, W = t.width;
  const uint32_t i0 = b * bag;
  const K id_mask = (K)(((uint64_t)1 << id_bits) - 1);
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC) {
    V acc;
    for (uint32_t h0 = 0; h0 < bag; h0 += kPoolAhead) {
      const embed_t *src[kPoolAhead];
#pragma unroll
      for (int k = 0; k < kPoolAhead; k++)
        src[k] = t.emb + (size_t)t.slot[(uint64_t)(keys[i0 + min(h0 + k, bag - 1)] & id_mask)] * W;
      V v[kPoolAhead];
#pragma unroll
      for (int k = 0; k < kPoolAhead; k++) v[k] = *(const V *)(src[k] + col);
#pragma unroll
      for (int k = 0; k < kPoolAhead; k++) {
        if (h0 + k == 0) acc = v[k];
        else if (h0 + k < bag) acc = acc + v[k];
      }
    }
    __builtin_nontemporal_store(acc, (V *)(dst_rows + (size_t)b * W + col));
  }
}

// plain 16-byte-lane copy of known size: the yardstick the HBM byte counters are scaled with
__global__ __launch_bounds__(kBlock) void plain_copy(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

inline int lanes_for(uint32_t width, int vec) {
  const uint32_t lanes = (width + vec - 1) / vec;
  return lanes <= 4 ? 4 : lanes <= 8 ? 8 : lanes <= 16 ? 16 : lanes <= 32 ? 32 : 64;
}

// expands F<VEC, LPR>(args...) over the supported (VEC, LPR) pairs
#define HCTR_DISPATCH_ROW(vec4, lpr, CALL) \
  do {                                     \
    if (vec4) {                            \
      switch (lpr) {                       \
        case 4: CALL(4, 4); break;         \
        case 8: CALL(4, 8); break;         \
        case 16: CALL(4, 16); break;       \
        case 32: CALL(4, 32); break;       \
        default: CALL(4, 64); break;       \
      }                                    \
    } else {                               \
      switch (lpr) {                       \
        case 4: CALL(1, 4); break;         \
        case 8: CALL(1, 8); break;         \
        case 16: CALL(1, 16); break;       \
        case 32: CALL(1, 32); break;       \
        default: CALL(1, 64); break;       \
      }                                    \
    }                                      \
  } while (0)

} // namespace

void launch_build_queries(hipStream_t s, const TableView &t, const KeyLayout &kl, const BatchView &cur, uint32_t unique_max,
                          const uint32_t *delta, index_t *q_idx, version_t *q_ver) {
  if (!unique_max) return;
  const dim3 grid(div_up(unique_max, kBlock)); // the kernel reads the number of unique keys itself
  if (kl.wide) hipLaunchKernelGGL(build_queries<uint64_t>, grid, dim3(kBlock), 0, s, t, kl.id_bits, cur, delta, q_idx, q_ver);
  else hipLaunchKernelGGL(build_queries<uint32_t>, grid, dim3(kBlock), 0, s, t, kl.id_bits, cur, delta, q_idx, q_ver);
  HCTR_HIP(hipGetLastError());
}

size_t query_tiles(uint32_t q) { return std::max<size_t>(1, div_up(q, kBlock)); }

uint32_t owner_push_rows_per_block(uint32_t width) {
  const int lpr = lanes_for(width, width % 4 == 0 ? 4 : 1);
  return kApplyBatches * kApplyAhead * (kBlock / lpr);
}

void launch_place_queries(hipStream_t s, OwnerShard *shards_dev, const OwnerShard *shards_host, int nsrc,
                          const QueryArea &area) {
  HCTR_CHECK(nsrc <= kBlock, "internal: more shards than the placing block has threads");
  PlaceSources src;
  for (int i = 0; i < kPlaceLds; i++) {
    src.send_cnt[i] = i < nsrc ? shards_host[i].send_cnt : nullptr;
    src.n_keys[i] = i < nsrc ? shards_host[i].n_keys : 0;
  }
  hipLaunchKernelGGL(place_queries, dim3(1), dim3(kBlock), 0, s, shards_dev, nsrc, area, src);
  HCTR_HIP(hipGetLastError());
}

// Grids of kernels whose work is known on the device only are cut from a guess (what the step before had, and some)
// and never beyond the most there can be; the kernels stride over what there is.
static uint32_t guessed_blocks(uint32_t guess, uint32_t most, uint32_t per_block) {
  const uint64_t g = (uint64_t)guess + guess / 4 + 4 * per_block;
  return std::max(1u, div_up(std::min<uint64_t>(g, most), per_block));
}

void launch_owner_side(hipStream_t s, const OwnerShard *shards_dev, int nshards, int nsrc, uint32_t width,
                       uint32_t push_blocks, uint32_t queries_max, uint32_t queries_guess) {
  const uint32_t tiles = guessed_blocks(queries_guess, queries_max, kBlock);
  const bool vec4 = width % 4 == 0;
  const int lpr = lanes_for(width, vec4 ? 4 : 1);
  if (push_blocks) {
    const uint32_t rpb = owner_push_rows_per_block(width);
#define CALL(V, L) \
  hipLaunchKernelGGL((apply_remote_all<V, L>), dim3(push_blocks, nshards), dim3(kBlock), 0, s, shards_dev, nsrc, rpb)
    HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  }
  hipLaunchKernelGGL(decide_count, dim3(tiles, nshards), dim3(kBlock), 0, s, shards_dev, nsrc);
  hipLaunchKernelGGL(scan_positions, dim3(tiles, nshards), dim3(kBlock), 0, s, shards_dev, nsrc);
  if (queries_max) {
    hipLaunchKernelGGL(place_returns, dim3(div_up((uint32_t)(nsrc * nsrc), kBlock)), dim3(kBlock), 0, s, shards_dev, nsrc);
#define CALL(V, L)                                                                                                     \
  hipLaunchKernelGGL((pack_rows<V, L>), dim3(guessed_blocks(queries_guess, queries_max, kPackAhead * (kBlock / L)), nshards), \
                     dim3(kBlock), 0, s, shards_dev, nsrc)
    HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  }
  HCTR_HIP(hipGetLastError());
}

void launch_refresh(hipStream_t s, const TableView &t, const BatchView &cur, uint32_t unique_max, uint32_t unique_guess,
                    const PullArgs &a, uint32_t *tile_sums, uint32_t *stats, uint32_t *host_stats) {
  if (!unique_max || !a.got) return;
  const unsigned tiles = div_up(unique_max, kRTile); // for the batch's keys; the kernels read how many are unique
  hipLaunchKernelGGL(got_tile_sums, dim3(tiles), dim3(kBlock), 0, s, a.got, cur.d_U, tile_sums);
  hipLaunchKernelGGL(remote_emit, dim3(tiles), dim3(kBlock), 0, s, t, cur, a.got, tile_sums, a.ret_i, a.src_row, stats,
                     host_stats);
  const bool vec4 = t.width % 4 == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
#define CALL(V, L)                                                                                                      \
  hipLaunchKernelGGL((refresh<V, L>), dim3(guessed_blocks(unique_guess, unique_max, kBlock / L)), dim3(kBlock), 0, s, t, cur, a)
  HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_gather(hipStream_t s, const TableView &t, const BatchView &cur, const PullArgs &a) {
  if (!cur.n) return;
  const bool vec4 = t.width % 4 == 0 && ((uintptr_t)a.dst % 16) == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
  const bool local_only = a.got == nullptr;
#define CALL(V, L)                                                                                               \
  do {                                                                                                           \
    const unsigned blocks = div_up(div_up(cur.n, kRows), kBlock / L);                                            \
    if (local_only && a.stream_stores) hipLaunchKernelGGL((gather<V, L, true, true>), dim3(blocks), dim3(kBlock), 0, s, t, cur, a); \
    else if (local_only) hipLaunchKernelGGL((gather<V, L, true, false>), dim3(blocks), dim3(kBlock), 0, s, t, cur, a); \
    else if (a.stream_stores) hipLaunchKernelGGL((gather<V, L, false, true>), dim3(blocks), dim3(kBlock), 0, s, t, cur, a); \
    else hipLaunchKernelGGL((gather<V, L, false, false>), dim3(blocks), dim3(kBlock), 0, s, t, cur, a);          \
  } while (0)
  HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_gather_direct(hipStream_t s, const TableView &t, const KeyLayout &kl, const void *keys, uint32_t n, embed_t *dst,
                          bool stream_stores) {
  if (!n) return;
  HCTR_CHECK(t.nrank == 1, "internal: the gather from the keys is for one shard");
  const bool vec4 = t.width % 4 == 0 && ((uintptr_t)dst % 16) == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
#define CALL(V, L)                                                                                                    \
  do {                                                                                                                \
    const unsigned blocks = div_up(n, (kBlock / L) * kRows);                                                          \
    if (kl.wide && stream_stores) hipLaunchKernelGGL((gather_direct<V, L, uint64_t, true>), dim3(blocks), dim3(kBlock), 0, s, t, (const uint64_t *)keys, kl.id_bits, n, dst); \
    else if (kl.wide) hipLaunchKernelGGL((gather_direct<V, L, uint64_t, false>), dim3(blocks), dim3(kBlock), 0, s, t, (const uint64_t *)keys, kl.id_bits, n, dst); \
    else if (stream_stores) hipLaunchKernelGGL((gather_direct<V, L, uint32_t, true>), dim3(blocks), dim3(kBlock), 0, s, t, (const uint32_t *)keys, kl.id_bits, n, dst); \
    else hipLaunchKernelGGL((gather_direct<V, L, uint32_t, false>), dim3(blocks), dim3(kBlock), 0, s, t, (const uint32_t *)keys, kl.id_bits, n, dst); \
  } while (0)
  HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_gather_pooled_direct(hipStream_t s, const TableView &t, const KeyLayout &kl, const void *keys, uint32_t n,
                                 embed_t *dst, uint32_t bag) {
  if (!n) return;
  HCTR_CHECK(t.nrank == 1, "internal: the gather from the keys is for one shard");
  const uint32_t n_bags = n / bag;
  const bool vec4 = t.width % 4 == 0 && ((uintptr_t)dst % 16) == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
#define CALL(V, L)                                                                                                    \
  do {                                                                                                                \
    const unsigned blocks = div_up(n_bags, kBlock / L);                                                               \
    if (kl.wide) hipLaunchKernelGGL((gather_pooled_direct<V, L, uint64_t>), dim3(blocks), dim3(kBlock), 0, s, t, (const uint64_t *)keys, kl.id_bits, dst, bag, n_bags); \
    else hipLaunchKernelGGL((gather_pooled_direct<V, L, uint32_t>), dim3(blocks), dim3(kBlock), 0, s, t, (const uint32_t *)keys, kl.id_bits, dst, bag, n_bags); \
  } while (0)
  HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_gather_pooled(hipStream_t s, const TableView &t, const BatchView &cur, const PullArgs &a, uint32_t bag) {
  if (!cur.n) return;
  const uint32_t n_bags = cur.n / bag;
  const bool vec4 = t.width % 4 == 0 && ((uintptr_t)a.dst % 16) == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
  const bool local_only = a.got == nullptr;
#define CALL(V, L)                                                                                                  \
  do {                                                                                                              \
    const unsigned blocks = div_up(n_bags, kBlock / L);                                                             \
    if (local_only) hipLaunchKernelGGL((gather_pooled<V, L, true>), dim3(blocks), dim3(kBlock), 0, s, t, cur, a, bag, n_bags); \
    else hipLaunchKernelGGL((gather_pooled<V, L, false>), dim3(blocks), dim3(kBlock), 0, s, t, cur, a, bag, n_bags);  \
  } while (0)
  HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_plain_copy(hipStream_t s, const void *src, void *dst, size_t bytes) {
  hipLaunchKernelGGL(plain_copy, dim3(256 * 16), dim3(kBlock), 0, s, (const uint4 *)src, (uint4 *)dst, bytes / 16);
  HCTR_HIP(hipGetLastError());
}

} // namespace hctr
