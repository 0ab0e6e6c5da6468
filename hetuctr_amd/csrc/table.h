// Host-side state of one shard (the reference's HetuTable, csrc/core/hetu_gpu_table.h:21-144) and of the
// in-process loopback group that stands in for the NCCL communicator.
#pragma once
#include <condition_variable>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/hetuctr_hip.h"
#include "host_copy.h"
#include "kernels.h"
#include "radix_sort.h"
#include "tile_sort.h"

namespace hctr {

// growable device allocation; contents are NOT kept when it grows
struct DeviceBuf {
  void *p = nullptr;
  size_t bytes = 0;
  DeviceBuf() = default;
  DeviceBuf(const DeviceBuf &) = delete;
  DeviceBuf &operator=(const DeviceBuf &) = delete;
  DeviceBuf(DeviceBuf &&o) noexcept : p(o.p), bytes(o.bytes) { o.p = nullptr; o.bytes = 0; }
  DeviceBuf &operator=(DeviceBuf &&o) noexcept {
    if (this != &o) {
      release();
      p = o.p;
      bytes = o.bytes;
      o.p = nullptr;
      o.bytes = 0;
    }
    return *this;
  }
  ~DeviceBuf() { release(); }
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    bytes = 0;
  }
  bool reserve(size_t want) { // true: a new allocation was made
    if (want <= bytes) return false;
    release();
    size_t grow = want + want / 8; // headroom so that slowly growing batches do not reallocate every step
    HCTR_HIP(hipMalloc(&p, grow));
    bytes = grow;
    return true;
  }
  template <typename T> T *as() const { return (T *)p; }
};

// per-batch buffers: the reference's PreprocessData (csrc/core/preprocess_struct.h:7-24)
struct Batch {
  uint32_t n = 0;   // keys
  uint32_t U = 0;   // unique keys (host copy, valid after the preprocess call returned)
  bool idx_map_valid = false;
  bool cleared = false; // the device side reads as an empty batch (U = 0, no buckets, no runs) since clear()
  bool planned = false; // the push plan (need, prefix, push_cnt) has been computed for the batch as it stands
  bool lists_ready = true;  // the run lists of the batch's push have been built (or the batch is empty)
  bool tile_sorted = false; // indexed by the tile-sorted passes (tile_sort.h)
  bool direct_gather = false; // one shard, small batch: the step's gather works from `comp` in batch order and does not
                              // wait for the index (the run lists are then built in front of the batch's push)
  bool comp_valid = false;    // comp holds the batch's sort keys in batch order
  bool keys_made = false;   // comp holds the batch's sort keys (a kernel of its own made them); else the first launch
                            // of the tile-sorted passes read the ids itself and no copy in batch order exists: the ids
                            // of the batch are read back through the index when somebody asks for them
  // comp: the batch's sort keys in batch order (id and owner of every position); staged: ids that arrived in
  // pageable host memory, on their way to the key kernel
  DeviceBuf comp, staged, sorted_arg, rank_sorted, idx_map, ukey, run_start, uoff, bucket_lo, dU, long_list, dnlong, med_list;
  DeviceBuf need, prefix, plan_total; // push plan per unique key: pushed or not, position among the pushed rows; their number
  std::vector<uint64_t> send_cnt, recv_cnt;       // queries per owner / per requester
  std::vector<uint64_t> push_cnt, pushrecv_cnt;   // pushed rows per owner / per source
  void reserve(uint32_t n_keys, int nrank, bool wide);
  bool holds(uint32_t n_keys, int nrank, bool wide) const; // reserve() would not allocate
  void clear(hipStream_t s, int nrank); // make the device side an empty batch; does nothing if it already is
  BatchView view() const;
};

// What the host reads back after a preprocess call: written by kernels into one device block (DevStat) and
// copied with ONE transfer into the pinned HostMirror.  A single shard only needs the first 16 bytes.
struct DevStat {
  uint32_t U;
  uint32_t err;
  uint32_t push_total;
  uint32_t pad;
  uint64_t send_cnt[257];
  uint64_t push_cnt[257];
};
struct HostMirror {
  DevStat st;
  uint32_t stats[4];
  uint32_t ret_seg[258];
  uint32_t key_err; // written by the kernel that reads the caller's ids when preprocess returns early (no copy)
};

class Group;

// launches of the sort that a deferred preprocess enqueues itself: the column scan and the scatter of the first pass
// and the count of the second (the first count comes from the key kernel); with the tile-sorted passes, the first of
// the launches that follow the key kernel
#ifndef HCTR_EARLY_SORT_STEPS
#define HCTR_EARLY_SORT_STEPS 4
#endif
#ifndef HCTR_EARLY_TILE_PASSES
#define HCTR_EARLY_TILE_PASSES 1
#endif
constexpr int kEarlySortSteps = HCTR_EARLY_SORT_STEPS, kEarlyTilePasses = HCTR_EARLY_TILE_PASSES;
// from this many keys on, a preprocess that returns early has its ids read by a kernel that only makes the sort keys
#ifndef HCTR_KEYS_FIRST_FROM
#define HCTR_KEYS_FIRST_FROM (1u << 20)
#endif
constexpr uint32_t kKeysFirstFrom = HCTR_KEYS_FIRST_FROM;
// One shard: a batch whose output rows take up to this many bytes is gathered in batch order straight from its keys
// (Batch::direct_gather).  Measured on an MI355X with 512-byte rows: 107 k keys 78 us per step against 92 with the gather
// in sorted order behind the index, 426 k keys 165 against 174, 852 k keys 316 against 279 -- in batch order the
// duplicates of a key are not adjacent, and from about the size of the last-level cache (256 MB) on the rows of a batch
// no longer stay cached between them.
#ifndef HCTR_DIRECT_GATHER_BYTES
#define HCTR_DIRECT_GATHER_BYTES (256ull << 20)
#endif

// stages whose device time can be measured separately (HIP events on the group's stream)
enum Stage { S_KEYS = 0, S_SORT, S_UNIQUE, S_PLAN, S_PUSH, S_QUERY, S_EXCHANGE, S_OWNER, S_REFRESH, S_GATHER, S_COUNT };
const char *stage_name(int s);

class Shard {
 public:
  Shard(const hctr_config &cfg, const uint8_t *root_arr, const int64_t *storage_arr, size_t n_storage,
        unsigned seed, std::shared_ptr<Group> group);
  ~Shard();

  hctr_config cfg;
  std::string ip;
  std::shared_ptr<Group> group;
  KeyLayout kl;
  TableView tv;
  size_t n_owned = 0;

  // ---- stages, each only enqueues on the group's stream (names follow hetu_gpu_table.h:82-97) ----
  void swap_batches() { std::swap(cur, prev); }
  void preprocess_index(const int64_t *keys, size_t n) {
    ingest_keys(keys, n);
    index_batch();
  }
  // the caller's ids -> device copy and sort keys; flag: where the range check reports (default: the device word)
  // scratch_area (default: the shard's own growable buffers): the index scratch of this batch is cut out of it
  void ingest_keys(const int64_t *keys, size_t n, uint32_t *flag = nullptr, void *scratch_area = nullptr);
  // sort, unique, run lists of the ingested batch; u_out: where the number of unique keys goes besides the batch's
  // own device word (default: the device block that is read back after the call)
  void index_batch(uint32_t *u_out = nullptr, int part = 0);
  TileSortBuffers tile_sort_buffers() const; // the index scratch as the tile-sorted passes take it
  HostStager stager;                         // ids that arrive in pageable host memory go through its pinned buffer
  bool pooled_from_keys = true;   // HETUCTR_POOLED_FROM_KEYS=0: pooled gathers of one shard go through the inverse index
  uint32_t direct_gather_max = 0; // keys: HCTR_DIRECT_GATHER_BYTES / bytes of a row, or HETUCTR_DIRECT_GATHER_MAX
  int tile_sort_mode = 1;                    // HETUCTR_TILE_SORT: 0 no batch takes the tile-sorted passes, 1 those of up
                                             // to kTileSortMaxKeys keys, 2 every batch whose tiles they can hold
  void plan_batch(Batch &b);  // enqueues the push plan of b; its counts reach the host when the stream has run it
  void enqueue_readback_preprocess();
  void finish_preprocess();                 // after the stream sync: mirrors -> host fields, error checks
  // the same in two halves, for a preprocess whose push plan and index run on different streams
  void finish_plan(Batch &b); // takes the counts over into b once they are there
  void finish_index();
  void check_key_error();                   // raises if the ingested batch held a key outside [0, length)
  // the push of a step in two halves, so that a group can place every shard's pushed rows before any push kernel runs
  void begin_push(const float *grad, uint32_t bag = 1);  // which batch is pushed (none on an inference step), checks
  void generate_gradient(const uint32_t *delta);         // the push kernel; delta: see Group::place_pushes
  void generate_query(const uint32_t *delta); // delta: see Group::place_queries
  // handleGradient + handleQuery: what the group's owner-side launches need of this shard (queries_max: no shard
  // receives more queries than this)
  void fill_owner_args(OwnerShard &o, uint64_t queries_max);
  void finish_handle_query();               // after the step: return counts and error flags from the pinned block
  void write_back(float *dst, uint32_t bag = 1);
  bool direct_now(uint32_t bag) const; // this step's gather works from the keys and does not wait for the index
  void finish_push_pull();

  size_t fetch(int which, void *host_out, size_t cap);
  // rows, versions, pending gradients and update counters to / from one file (checkpoint.hip)
  void save(const char *path);
  void load(const char *path);

  Batch cur, prev;
  bool prev_active = false; // false: inference step or no previous batch, nothing is pushed
  DeviceBuf root, slot, emb, ver, pend, upd, store_ids;
  // scratch shared by the stages
  DeviceBuf ktmp0, ktmp1, vtmp0, vtmp1, sortws, block_sums, headws, dstat, stats;
  // where the index stages of the current batch find their scratch: the buffers above or pieces of the static array
  struct ScratchPtrs {
    void *ktmp0 = nullptr, *ktmp1 = nullptr;
    uint32_t *vtmp0 = nullptr, *vtmp1 = nullptr, *sortws = nullptr, *block_sums = nullptr, *headws = nullptr;
  } sp;
  DeviceBuf plan_sums, query_sums; // query_sums: flags per tile of received queries // plan_sums: scan scratch of the push plan (the index has block_sums to itself)
  DevStat *dst_ = nullptr; // == dstat.p
  uint32_t *err_ptr() const { return &dst_->err; }
  // send side
  const float *push_grad_ = nullptr; // arguments of the push between begin_push and generate_gradient
  uint32_t push_bag_ = 1;
  // receive side (owner role)
  DeviceBuf src_row, ret_seg_dev;
  std::vector<uint64_t> rq_seg, rg_seg, ret_seg; // R+1 prefix offsets per source / requester
  uint64_t rg_base = 0;      // first row of this shard's piece of the group's receive area for pushed rows
  uint64_t rq_base = 0;      // first query of its piece of the receive area for queries (rq_seg, rq_base: the host's
                             // copy of what place_queries computed on the device, made when the step is over)
  DeviceBuf push_pos;        // place of every unique key's pushed row in that area (plan position + distance)
  // requester side of the return
  DeviceBuf got, ret_i, in_ver, in_val;
  HostMirror *mirror = nullptr;
  long long last_stats[6] = {0, 0, 0, 0, 0, 0};
  float last_pre_ms = 0.f, last_pp_ms = 0.f, last_push_ms = 0.f;
  bool u_cleared = false;    // the device-side copy of the number of unique keys reads as zero

 private:
  void reserve_batch_scratch(uint32_t n);
  void use_scratch_area(void *area, uint32_t n);
};

// The entry point that allocates nothing takes batches of up to kNoAllocMaxKeys keys; kNoAllocScratchBytes is what
// the index of such a batch needs with 64-bit sort keys (sort ping-pong buffers, per-tile digit tables, scan sums, head
// counts per chunk), every piece rounded up to 256 bytes.
constexpr size_t kNoAllocMaxKeys = 262144;
constexpr size_t index_scratch_round(size_t b) { return (b + 255) / 256 * 256; }
// words of digit tables either sort of a batch of n keys needs
constexpr inline size_t index_table_words(size_t n) {
  const size_t a = sort_scratch_words(n), b = tile_sort_possible(n) ? tile_sort_table_words(n) : 0;
  return a > b ? a : b;
}
// bytes of index scratch a batch of n keys needs (n >= 1)
constexpr inline size_t index_scratch_bytes(uint32_t n, bool wide) {
  const size_t m = n < 1 ? 1 : n, ks = wide ? 8 : 4;
  return 2 * index_scratch_round(m * ks) + 2 * index_scratch_round(m * 4) + index_scratch_round(index_table_words(m) * 4) +
         index_scratch_round((scan_blocks(m) + 2) * 4) + index_scratch_round(head_chunk_words(m) * 4);
}
// An upper bound of index_scratch_bytes over all n <= kNoAllocMaxKeys that needs no loop: the tables of the smallest
// tile shape (or of the most tiles the tile-sorted passes take) and the head counts of the smallest chunk at the largest n.
constexpr size_t kNoAllocScratchBytes =
    2 * (kNoAllocMaxKeys * 8) + 2 * (kNoAllocMaxKeys * 4) +
    (kNoAllocMaxKeys / (kSortBlock * kSortItemsSmall) + 8) * kSortMaxBins * 4 + (kNoAllocMaxKeys / 2048 + 3) * 4 +
    (kNoAllocMaxKeys / 128 + 1) * 5 * 4 + 64 + 8 * 256;
static_assert((kTileSortMaxTiles + 7) / 8 * 8 <= kNoAllocMaxKeys / (kSortBlock * kSortItemsSmall) + 8, "tables of the tile-sorted passes");
// the sizes where the tile shape of a sort changes, and the largest batch: changed tile constants fail here
static_assert(index_scratch_bytes((uint32_t)kSortSmallUpTo, true) <= kNoAllocScratchBytes &&
                  index_scratch_bytes((uint32_t)kSortSmallUpTo + 1, true) <= kNoAllocScratchBytes &&
                  index_scratch_bytes((uint32_t)(2 * kTileSortMaxTiles * kSortBlock), true) <= kNoAllocScratchBytes &&
                  index_scratch_bytes((uint32_t)(2 * kTileSortMaxTiles * kSortBlock) + 1, true) <= kNoAllocScratchBytes &&
                  index_scratch_bytes((uint32_t)kNoAllocMaxKeys, true) <= kNoAllocScratchBytes,
              "the static scratch of the entry point that allocates nothing is too small");

// All shards of one loopback group live in one process on one device and share one stream.  The group
// carries the collective calls: every shard's thread deposits its arguments, the last one to arrive runs the
// step for all shards, the others wait for it.
class Group {
 public:
  Group(int nrank, int device_id, std::string key);
  ~Group();
  const int nrank;
  const int device_id;
  const std::string key;
  hipStream_t stream = nullptr;          // the stream the stages enqueue on (see StreamSwitch)
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  // Single shard: preprocess enqueues its work on a second stream and returns once the caller's ids are consumed;
  // sorting and deduplicating them has no dependence on the pending gradient push, so the next push_pull starts the
  // push on the main stream right away and only the gather waits for both.
  hipStream_t index_stream = nullptr;
  hipEvent_t ev_index = nullptr, ev_keys = nullptr, ev_push = nullptr, ev_pushed = nullptr, ev_plan = nullptr;
  bool defer_index = false;              // the mode is on (HETUCTR_DEFER_INDEX != 0)
  bool index_pending = false;            // a batch's index is enqueued and nobody has waited for it yet
  bool index_rest_pending = false;       // single shard: preprocess enqueued only the first launches of the index
  void enqueue_index_rest();
  void enqueue_index_all(int part);             // enqueues the others
  void flush_index();                    // waits for a pending index and takes its results over
  // owner-side arguments of every shard: pinned staging and the device copy the kernels read
  OwnerShard *owner_host = nullptr;
  DeviceBuf owner_dev, ret_delta_dev;    // ret_delta_dev: nrank words per owner, see OwnerShard::ret_delta
  void owner_side(uint64_t queries_max);
  // Where every shard's pushed rows go: one receive area for the whole group (ids, counts, rows), cut into one piece
  // per owner and, inside it, per source; sized from the plans before any push kernel runs.  Every sender gets, per
  // owner, the distance between a row's place in its own plan and its place in the area (nrank words per sender).
  void place_pushes();
  DeviceBuf rg_idx_all, rg_cnt_all, rg_val_all, push_delta_dev;
  uint32_t *push_delta_host = nullptr;   // pinned staging of the distances
  // The same for the queries of a step: one receive area (ids, versions, and what the owners keep per query), nrank
  // distances per requester.  How many queries go where is known on the device only: reserve_queries() sizes the area
  // for the most there can be, launch_place_queries (behind the upload of the owners' records) cuts it.
  uint64_t reserve_queries();
  QueryArea query_area();
  void note_query_places(); // rq_seg / rq_base of every shard from the counts the host has once the step is over
  uint32_t queries_guess_ = 0; // queries the busiest owner received in the step before
  bool queries_seen_ = false;
  DeviceBuf rq_idx_all, rq_ver_all, rq_outdated_all, rq_slot_all, rq_ret_all, query_delta_dev;
  bool time_calls = false;               // bracket the two calls with events (hctr_call_timing)
  std::vector<Shard *> members;
  double wait_seconds = 120.0;
  void sync_stream();

  // per-stage device time, accumulated over calls while stage_timing is on
  bool stage_timing = false;
  double stage_ms[S_COUNT] = {};
  long long stage_calls[S_COUNT] = {};
  struct StageMark { int stage; hipEvent_t a, b; };
  std::vector<StageMark> marks;          // of the call in flight
  std::vector<hipEvent_t> event_pool;
  hipEvent_t take_event();
  void collect_marks();                  // after a stream sync
  void set_defer_index(bool on);         // switches the early return of preprocess; waits for a pending index first
  void set_call_timing(bool on);         // events around the two calls; the times of earlier calls are forgotten
  void set_stage_timing(bool on);        // resets the accumulators; waits for a pending index under the group's lock

  void join(Shard *s);
  void leave(Shard *s);
  bool complete() const;

  // lock-step bodies (one caller)
  void preprocess_all(const int64_t *const *keys, const size_t *n);
  void preprocess_noalloc(const int64_t *keys, size_t n);
  void *noalloc_scratch = nullptr;       // device address of this GPU's static scratch array
  // bag > 1: sum-pooled lookups, grads and dsts hold one row per bag of `bag` consecutive keys
  void push_pull_all(const float *const *grads, float *const *dsts, size_t bag = 1);
  // per-shard entry points: rendezvous of nrank callers
  void preprocess_one(int rank, const int64_t *keys, size_t n);
  void push_pull_one(int rank, const float *grad, float *dst, size_t bag = 1);

 private:
  void exchange_shapes();
  void push_pull_steps(const float *const *grads, float *const *dsts, uint32_t bag); // the body of push_pull_all
  bool index_joining_ = false; // push_pull has taken a pending index over and not yet read its results
  template <typename F> void collective(int rank, int op, F &&run_all);
  std::mutex mu_;
  std::condition_variable cv_;
  int arrived_ = 0, pending_op_ = 0;
  uint64_t generation_ = 0;
  std::string failure_;
  std::vector<const int64_t *> a_keys_;
  std::vector<size_t> a_n_;
  std::vector<const float *> a_grad_;
  std::vector<float *> a_dst_;
  std::vector<size_t> a_bag_;
};

// brackets the launches of one stage with two events when stage timing is on
struct StageScope {
  Group &g;
  int idx = -1;
  StageScope(Group &grp, int stage) : g(grp) {
    if (!g.stage_timing) return;
    Group::StageMark m{stage, g.take_event(), g.take_event()};
    HCTR_HIP(hipEventRecord(m.a, g.stream));
    g.marks.push_back(m);
    idx = (int)g.marks.size() - 1;
  }
  ~StageScope() {
    if (idx >= 0) (void)hipEventRecord(g.marks[idx].b, g.stream);
  }
};

// makes the stages enqueue on another stream for the lifetime of the object
struct StreamSwitch {
  Group &g;
  hipStream_t saved;
  StreamSwitch(Group &grp, hipStream_t s) : g(grp), saved(grp.stream) { g.stream = s; }
  ~StreamSwitch() { g.stream = saved; }
};

std::shared_ptr<Group> find_or_create_group(int nrank, int device_id, const std::string &ip, int port);

} // namespace hctr
