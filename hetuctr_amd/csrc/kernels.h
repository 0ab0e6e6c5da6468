// Host-callable launchers of the hot-path kernels.  Each one only enqueues work on `stream`.
// Reference stages are cited where the launcher is defined.
#pragma once
#include "common.h"

namespace hctr {

// The sort key of a batch position: (owner << id_bits) | id.  Its order is the reference's
// id + kEmbeddingIDMax*owner (csrc/core/preprocess.cu:17): owner first, id second.
struct KeyLayout {
  int id_bits;    // bits of an id
  int total_bits; // id_bits + bits of an owner
  bool wide;      // 64-bit sort keys (total_bits > 32)
  int max_digit_bits = 0; // widest digit of the tile-sorted passes (0: the most the sort takes); narrower for tests
};

// Device-side view of one preprocessed batch (the reference's PreprocessData,
// csrc/core/preprocess_struct.h:7-24, with 32-bit positions and ranks).
struct BatchView {
  uint32_t n;                // keys in the batch (host-known)
  uint32_t *sorted_arg;      // [n]   positions grouped by unique key, stable   (d_sorted_arg)
  uint32_t *rank_sorted;     // [n]   unique rank of sorted position j
  uint32_t *idx_map;         // [n]   unique rank of position i, filled on request only    (d_idx_map)
  void *ukey;                // [U]   sort key of unique rank u: id and owner   (d_unique_idx, d_root)
  uint32_t *run_start;       // [U+1] first sorted position of rank u           (d_run_length)
  slot_t *uoff;              // [U]   resident offset of rank u or -1           (d_offset)
  uint32_t *bucket_lo;       // [R+1] first rank owned by each shard            (u_shape before :131)
  uint32_t *d_U;             // [1]   number of unique keys                     (unique_size)
  uint4 *long_list;          // [kLongBuckets][long_cap] runs longer than kLongRun by length class: {unique rank, first sorted position, length, resident offset}
  uint32_t *d_nlong;         // [kRunCounters] entries per class of long runs, then counters of the push
  uint32_t long_cap;         // capacity of one class
  uint32_t *med_list;        // [d_nlong[kMedCount]] unique ranks with kTinyRun < run length <= kLongRun (any order)
};

// d_nlong layout: [0, kLongBuckets) long runs per class, then the number of medium runs and the ticket counters of
// the long role
constexpr int kLongBuckets = 12;
constexpr int kMedCount = kLongBuckets, kTicketBase = kLongBuckets + 1, kTicketLanes = 16,
              kRunCounters = kTicketBase + 2 * kTicketLanes;

// A run of equal keys longer than this is summed by a whole block that streams its gradient rows through
// LDS; shorter runs are summed by a small group of lanes.
#ifndef HCTR_LONG_RUN
#define HCTR_LONG_RUN 128
#endif
constexpr uint32_t kLongRun = HCTR_LONG_RUN;
#ifndef HCTR_TINY_RUN
#define HCTR_TINY_RUN 8
#endif
constexpr uint32_t kTinyRun = HCTR_TINY_RUN; // runs up to this length are summed by the group that owns their rank
// Long runs are listed by length class (class 0 = longest) so that the push can start the longest chains first.
inline size_t long_list_capacity(uint32_t n) { return n / (kLongRun + 1) + 1; }
inline size_t med_list_capacity(uint32_t n) { return n / (kTinyRun + 1) + 1; }
__host__ __device__ inline int long_bucket(uint32_t len) {
  // class c holds lengths in [2^(17-c), 2^(18-c)), the first everything from 2^17 up, the last everything below 256
  int c = 0;
  for (uint32_t lim = 1u << 17; c < kLongBuckets - 1 && len < lim; lim >>= 1) c++;
  return c;
}

struct TableView {
  int rank, nrank;
  uint64_t id_max;
  uint32_t width;
  uint32_t n_stored, n_cached;   // kStorageMax, kNonLocalStorageMax
  float neg_lr;
  version_t pull_bound, push_bound;
  const worker_t *root;          // [id_max]
  const slot_t *slot;            // [id_max]  id -> resident offset or -1
  embed_t *emb;                  // [n_stored][width]
  version_t *ver;                // [n_stored]
  embed_t *pend;                 // [n_cached][width]
  version_t *upd;                // [n_cached]
};

// ---- preprocess ---------------------------------------------------------------------------------
// ids -> sort keys; flags ids outside [0, id_max) in *err (and sorts them as id 0)
// comp_keys is the batch's copy of the ids as well (the reference's d_idx); nlong (optional) is zeroed;
// sort_counts: the sort's scratch, which receives the per-tile counts of the first pass' digit
// ids32: `keys` points to 32-bit ids (narrowed on their way from pageable host memory; one that did not fit is
// 0xffffffff, which the range check flags like the id it stands for)
void launch_make_keys(hipStream_t s, const TableView &t, const KeyLayout &kl, const index_t *keys, uint32_t n,
                      void *comp_keys, uint32_t *err, uint32_t *nlong, uint32_t *sort_counts, bool ids32 = false);
// sorted keys -> everything per unique key + inverse index.  heads: the head counts per chunk of sorted positions that
// the last launch of the tile-sorted passes left (count_heads false), or storage for them (count_heads true: a launch
// of its own counts them first, one chunk per tile of the unique pass).
// u_copy (optional) receives the number of unique keys as well (b.d_U always does)
struct HeadChunks;
void launch_unique(hipStream_t s, const TableView &t, const KeyLayout &kl, const void *sorted_keys,
                   const BatchView &b, const HeadChunks &heads, bool count_heads, uint32_t *u_copy);

// batch-order inverse index from sorted_arg and rank_sorted (introspection; the hot path does not need it)
void launch_idx_map(hipStream_t s, const BatchView &b);
// the run lists of the batch (run_lists.h) by a launch of their own, after launch_unique; the gather builds them on its
// way when PullArgs::list_chunks is set
void launch_list_long_runs(hipStream_t s, const BatchView &b);
inline uint32_t run_list_chunks(uint32_t n) { return (n + 255) / 256; } // enough for any number of unique keys <= n

// device-wide exclusive scan of n (<= *d_n if d_n != nullptr) 32-bit values; block_sums: div_up(n_max,2048)+1 words.
// total (optional) receives the sum.
void launch_exclusive_scan(hipStream_t s, const uint32_t *in, uint32_t *out, uint32_t n_max, const uint32_t *d_n,
                           uint32_t *block_sums, uint32_t *total);

// push plan of the previous batch (csrc/core/preprocess.cu:148-165): need[u] in {0,1}
void launch_decide_update(hipStream_t s, const TableView &t, const KeyLayout &kl, const BatchView &prev,
                          uint32_t *need);
// pushed rows per owner from the scanned plan: cnt[d] = prefix[lo[d+1]] - prefix[lo[d]]
void launch_bucket_counts(hipStream_t s, const BatchView &b, const uint32_t *prefix, const uint32_t *total,
                          int nrank, uint64_t *cnt_out, uint64_t *host_out);
// both also write their counts to host_out (pinned host memory), bucket_sizes the number of unique keys to host_U
void launch_bucket_sizes(hipStream_t s, const BatchView &b, int nrank, uint64_t *cnt_out, uint64_t *host_out,
                         uint32_t *host_U);

// Division of a batch position by the bag size of sum-pooled lookups without a divide instruction: for any 32-bit
// n and bag >= 2, n / bag == (((n - q) >> 1) + q) >> shift with q = high word of n * magic (the "round up, add back"
// form of division by an invariant integer).  bag == 1 leaves positions alone (no shifts, magic 0).
struct BagDiv {
  uint32_t bag = 1, magic = 0, half = 0, shift = 0;
  BagDiv() = default;
  explicit BagDiv(uint32_t d) : bag(d) {
    if (d < 2) return; // magic 0 and no shifts: the formula below returns n
    half = 1;
    int lg = 31;
    while (!((d >> lg) & 1u)) lg--; // floor(log2 d)
    if ((d & (d - 1)) == 0) {         // a power of two: q is 0 and the two shifts make up log2(d)
      magic = 0;
      shift = (uint32_t)lg - 1;
      return;
    }
    const uint64_t num = (uint64_t)1 << (32 + lg);
    uint64_t m = num / d;
    const uint64_t rem = num - m * d;
    m = (m + m) & 0xffffffffull;
    const uint64_t twice = rem + rem;
    if (twice >= d) m += 1;
    magic = (uint32_t)(m + 1);
    shift = (uint32_t)lg;
  }
  // straight-line code for every bag size (a branch here would sit inside the load pipelines of the push)
  __host__ __device__ __forceinline__ uint32_t operator()(uint32_t n) const {
#ifdef __HIP_DEVICE_COMPILE__
    const uint32_t q = __umulhi(n, magic);
#else
    const uint32_t q = (uint32_t)(((uint64_t)n * magic) >> 32);
#endif
    return (((n - q) >> half) + q) >> shift;
  }
};

// ---- push: segment-sum of gradients by unique key + fused SGD ----------------------------------------
struct PushArgs {
  const embed_t *grad;       // [n_prev / bag][width]
  BagDiv bag;                // bag size of sum-pooled lookups (1: none): position i reads gradient row i / bag
  const uint32_t *need;      // [U_prev] or nullptr when nrank == 1
  const uint32_t *prefix;    // [U_prev] push slot
  index_t *g_idx;            // push buffers
  version_t *g_cnt;
  embed_t *g_val;
};
// pos[u] = prefix[u] + delta[owner of unique key u] for the n_unique unique keys of `prev`: the place of a pushed row in
// a receive area shared by all owners, from its place in the shard's own plan (delta: nrank words in device memory)
void launch_place_rows(hipStream_t s, const KeyLayout &kl, const BatchView &prev, uint32_t n_unique,
                       const uint32_t *prefix, const uint32_t *delta, uint32_t *pos);
// n_unique: number of unique keys of `prev` (host copy)
void launch_push(hipStream_t s, const TableView &t, const KeyLayout &kl, const BatchView &prev, uint32_t n_unique,
                 const PushArgs &a);

// ---- query / owner side / pull -------------------------------------------------------------------------
// id and local version of every unique key of the current batch, written to place (unique rank + delta[owner of the
// key]) of q_idx / q_ver (delta: nrank words in device memory).  unique_max: no more unique keys than this (the batch's
// size); how many there are the kernel reads from cur.d_U.
void launch_build_queries(hipStream_t s, const TableView &t, const KeyLayout &kl, const BatchView &cur, uint32_t unique_max,
                          const uint32_t *delta, index_t *q_idx, version_t *q_ver);
// Owner side of a step: applying the received pushes (per target row in source order) and serving the received
// queries (outdated flags, positions of the rows to return, rows packed, first returned row of every requester).
// One entry per shard of the group; one set of launches serves them all.
struct OwnerShard {
  TableView t;
  // received pushes, sources concatenated in rank order; rg_seg[0..nsrc]: first row of every source
  const index_t *rg_idx;
  const version_t *rg_cnt;
  const embed_t *rg_val;
  uint32_t rg_seg[258];
  int longest;               // the source with the most rows
  uint32_t push_blocks;      // blocks the push kernel needs for this shard (rows of `longest` / rows per block)
  // Received queries; rq_seg[0..nsrc]: first query of every requester; [rq_seg[rank], rq_seg[rank + 1]) are its own.
  // How many unique keys every shard asks every owner for is known on the device only (the host does not wait for the
  // index of the current batches): send_cnt / n_keys are filled in on the host, and place_queries -- a launch in front
  // of the query kernels -- cuts the group's receive area from them and writes rq_idx .. ret_slot and got_delta below.
  const uint64_t *send_cnt;  // [nsrc] unique keys of THIS shard's current batch per owner (written by its index)
  uint32_t n_keys;           // keys of this shard's current batch; 0: the shard asks for nothing (send_cnt is stale)
  const index_t *rq_idx;
  const version_t *rq_ver;
  uint32_t rq_seg[258];
  uint32_t q, query_tiles;
  uint32_t *outdated, *tile_cnt;
  slot_t *q_slot;            // slot of every received query (kNoSlot: not owned here)
  slot_t *ret_slot;          // slots of the rows to return, in return order
  // The returned rows are written straight into the requesters' buffers.  in_ver / in_val: THIS shard's buffers as a
  // requester (an owner finds its requester s in entry s of the array of shards); ret_delta[s]: what an owner adds to
  // the place of a row in its own return order to get the row's place in requester s' buffers, where the rows of all
  // owners stand in owner order.
  version_t *in_ver;
  embed_t *in_val;
  uint32_t *ret_delta;       // [nsrc]
  // The flag of every received query goes straight to its requester as well: got = THIS shard's flags as a requester
  // (one per unique key, owners in rank order); got_delta[s]: what an owner adds to the place of a query in its receive
  // buffer to get the place of the flag in requester s' array (written by place_queries).
  uint32_t *got;
  uint32_t got_delta[257];
  uint32_t *err;             // the shard's error word
  uint32_t *seg_dev;         // [0..nsrc] first returned row of every requester's segment, device copy
  uint32_t *seg_host;        // the same in memory the host reads; [257] = error flags
};
size_t query_tiles(uint32_t q);                       // tile_cnt needs this many words + 1
uint32_t owner_push_rows_per_block(uint32_t width);   // rows of the longest source one block of the push kernel takes
// The receive area of the queries of a step, shared by all owners of the group: every array holds one entry per unique
// key of all current batches at most (`capacity`).  launch_place_queries cuts it: one piece per owner, inside it one per
// requester, both in rank order (csrc/core/all2all.cu:18-46), from the counts the shards' index kernels left on the
// device, and writes into every shard's record where its piece lies, and into query_delta[s * nsrc + d] what requester
// s adds to the rank of a unique key owned by d to get the key's place in the area.
struct QueryArea {
  index_t *idx;
  version_t *ver;
  uint32_t *outdated;
  slot_t *q_slot, *ret_slot;
  uint32_t *query_delta;     // [nsrc * nsrc]
};
// (shards_host: the records as the host filled them in, for the addresses of the counts)
void launch_place_queries(hipStream_t s, OwnerShard *shards_dev, const OwnerShard *shards_host, int nsrc,
                          const QueryArea &area);
// shards_dev: the array in device memory.  nshards == nsrc: every shard of the group is in the array, in rank order (an
// owner looks its requesters up there).  push_blocks: the most blocks a shard's received pushes need; queries_max: no
// shard receives more queries than this; queries_guess: what the busiest shard probably receives (the grids are cut
// from it; what a shard does receive, the kernels read from the records and stride over).
void launch_owner_side(hipStream_t s, const OwnerShard *shards_dev, int nshards, int nsrc, uint32_t width,
                       uint32_t push_blocks, uint32_t queries_max, uint32_t queries_guess);
// requester: refresh cached rows that came back, then gather every key's row into dst
struct PullArgs {
  const uint32_t *got;       // [U] or nullptr: nothing came back (nrank == 1)
  uint32_t *ret_i;           // [U] index into the returned rows (written by launch_refresh)
  uint32_t *src_row;         // [U] where the gather reads a key's row (written by launch_refresh): offset or returned row
  const version_t *in_ver;
  const embed_t *in_val;
  embed_t *dst;              // [n][width]
  bool stream_stores;        // write dst with nontemporal stores (see Shard::write_back)
  uint32_t list_chunks;      // the gather also builds the batch's run lists (run_lists.h): chunks of unique ranks, else 0
};
// Index of every returned row per unique key (a.ret_i), where the gather reads each key's row (a.src_row), the counts of
// the step and the refresh of the cached rows that came back.  tile_sums: scratch of scan_blocks(unique_max) words (unique_max: the batch's size; the number of unique keys is read from cur.d_U; unique_guess: the grid of the row kernel is cut from it);
// stats: five device words that read zero before the first call (the launch leaves them zero again); host_stats: four
// words the device can write (hit / miss / refreshed counts of the step, error bits)
void launch_refresh(hipStream_t s, const TableView &t, const BatchView &cur, uint32_t unique_max, uint32_t unique_guess,
                    const PullArgs &a,
                    uint32_t *tile_sums, uint32_t *stats, uint32_t *host_stats);
void launch_gather(hipStream_t s, const TableView &t, const BatchView &cur, const PullArgs &a);
// one shard: dst[i] = row of the id in keys[i] (the batch's sort keys in batch order), for all n positions; needs
// nothing of the batch's index
void launch_gather_direct(hipStream_t s, const TableView &t, const KeyLayout &kl, const void *keys, uint32_t n, embed_t *dst,
                          bool stream_stores);
// the same for bags of `bag` consecutive positions, one summed output row per bag (n a multiple of bag)
void launch_gather_pooled_direct(hipStream_t s, const TableView &t, const KeyLayout &kl, const void *keys, uint32_t n,
                                 embed_t *dst, uint32_t bag);
// sum-pooled lookups: dst[b] = the rows of positions b * bag .. b * bag + bag - 1 added up in that order
// (cur.idx_map must be filled: launch_idx_map)
void launch_gather_pooled(hipStream_t s, const TableView &t, const BatchView &cur, const PullArgs &a, uint32_t bag);

// ---- init -------------------------------------------------------------------------------------------------
void launch_init_values(hipStream_t s, embed_t *out, size_t len, int type, float a, float b, unsigned seed);
void launch_fill_i64(hipStream_t s, version_t *p, size_t n, version_t v);
void launch_fill_i32(hipStream_t s, int32_t *p, size_t n, int32_t v);
void launch_build_directory(hipStream_t s, const index_t *store_ids, uint32_t n_stored, slot_t *slot);
void launch_plain_copy(hipStream_t s, const void *src, void *dst, size_t bytes); // bytes % 16 == 0
// keys_out[r * fields + f] = log[rows[r] * fields + f]; a row number outside [0, n_samples) sets bit 0 of *err
void launch_sample_rows(hipStream_t s, const index_t *log, uint64_t n_samples, uint32_t fields, const index_t *rows,
                        uint64_t n_rows, index_t *keys_out, uint32_t *err);

} // namespace hctr
