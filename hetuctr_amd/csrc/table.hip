// Host orchestration of the hot path: shard construction, the fixed stage order of preprocess and push_pull,
// the placement of what the shards of a loopback group hand to each other, introspection.
// Reference: csrc/core/hetu_gpu_table.cu:9-65 (stage order), csrc/core/table_initialize.cu:66-211 (state),
// csrc/core/all2all.cu:6-130 (what travels between which buffers, in which order).
#include "table.h"

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <map>

namespace hctr {

const char *stage_name(int s) {
  static const char *names[S_COUNT] = {"make_keys", "radix_sort", "unique_emit", "push_plan", "segment_sum_apply",
                                       "query_build", "exchange", "owner_side", "cache_refresh", "gather"};
  return s >= 0 && s < S_COUNT ? names[s] : "?";
}

// ---- scratch of the entry point that allocates nothing (hctr_preprocess_noalloc) --------------------------------
// One array per GPU, held from the moment the library is loaded on it until the process ends.  In host code the
// array's name is only a handle: the device address comes from hipGetSymbolAddress, once per device, and that pointer
// is what kernels and copies are given.
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {
std::mutex g_scratch_mu;
std::map<int, void *> g_scratch_ptr; // device ordinal -> address of that device's copy of `scratch`
} // namespace

// address of the current device's copy of the array (dev must be the current device)
static void *noalloc_scratch_of(int dev) {
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  auto it = g_scratch_ptr.find(dev);
  if (it != g_scratch_ptr.end()) return it->second;
  void *ptr = nullptr;
  HCTR_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
  HCTR_CHECK(ptr != nullptr, "no device address for the static scratch array");
  g_scratch_ptr[dev] = ptr;
  return ptr;
}

static int bits_for(uint64_t max_value) { // bits needed to represent values 0..max_value
  int b = 0;
  while (b < 64 && (max_value >> b)) b++;
  return b;
}

// ================================================================================================
// Batch
// ================================================================================================
bool Batch::holds(uint32_t n_keys, int nrank, bool wide) const {
  const size_t n = std::max<uint32_t>(n_keys, 1);
  return comp.bytes >= n * (wide ? 8 : 4) && sorted_arg.bytes >= n * 4 && rank_sorted.bytes >= n * 4 &&
         idx_map.bytes >= n * 4 && ukey.bytes >= n * (wide ? 8 : 4) && run_start.bytes >= (n + 1) * 4 &&
         uoff.bytes >= n * sizeof(slot_t) && bucket_lo.bytes >= (size_t)(nrank + 1) * 4 && dU.bytes >= 4 &&
         long_list.bytes >= long_list_capacity((uint32_t)n) * sizeof(uint4) * kLongBuckets &&
         dnlong.bytes >= 4 * kRunCounters && med_list.bytes >= med_list_capacity((uint32_t)n) * 4;
}

void Batch::reserve(uint32_t n_keys, int nrank, bool wide) {
  const size_t n = std::max<uint32_t>(n_keys, 1);
  comp.reserve(n * (wide ? 8 : 4));
  sorted_arg.reserve(n * 4);
  rank_sorted.reserve(n * 4);
  idx_map.reserve(n * 4);
  ukey.reserve(n * (wide ? 8 : 4));
  bool fresh = run_start.reserve((n + 1) * 4);
  uoff.reserve(n * sizeof(slot_t));
  fresh |= bucket_lo.reserve((size_t)(nrank + 1) * 4);
  fresh |= dU.reserve(4);
  long_list.reserve(long_list_capacity((uint32_t)n) * sizeof(uint4) * kLongBuckets);
  fresh |= dnlong.reserve(4 * kRunCounters);
  med_list.reserve(med_list_capacity((uint32_t)n) * 4);
  if (fresh) cleared = false;
}

void Batch::clear(hipStream_t s, int nrank) {
  if (cleared) return;
  HCTR_HIP(hipMemsetAsync(dU.p, 0, 4, s));
  HCTR_HIP(hipMemsetAsync(bucket_lo.p, 0, (size_t)(nrank + 1) * 4, s));
  HCTR_HIP(hipMemsetAsync(run_start.p, 0, 4, s));
  HCTR_HIP(hipMemsetAsync(dnlong.p, 0, 4 * kRunCounters, s));
  cleared = true;
}

BatchView Batch::view() const {
  BatchView v;
  v.n = n;
  v.sorted_arg = sorted_arg.as<uint32_t>();
  v.rank_sorted = rank_sorted.as<uint32_t>();
  v.idx_map = idx_map.as<uint32_t>();
  v.ukey = ukey.p;
  v.run_start = run_start.as<uint32_t>();
  v.uoff = uoff.as<slot_t>();
  v.bucket_lo = bucket_lo.as<uint32_t>();
  v.d_U = dU.as<uint32_t>();
  v.long_list = long_list.as<uint4>();
  v.d_nlong = dnlong.as<uint32_t>();
  v.long_cap = (uint32_t)long_list_capacity(std::max<uint32_t>(n, 1));
  v.med_list = med_list.as<uint32_t>();
  return v;
}

// ================================================================================================
// Shard
// ================================================================================================
Shard::Shard(const hctr_config &c, const uint8_t *root_arr, const int64_t *storage_arr, size_t n_storage,
             unsigned seed, std::shared_ptr<Group> grp)
    : cfg(c), ip(c.ip ? c.ip : ""), group(std::move(grp)) {
  cfg.ip = nullptr;
  HCTR_CHECK(c.nrank >= 1 && c.nrank <= 256, "nrank must be in 1..256 (worker ids are one byte)");
  HCTR_CHECK(c.rank >= 0 && c.rank < c.nrank, "rank out of range");
  HCTR_CHECK(c.length >= 1, "length must be positive");
  HCTR_CHECK(c.width >= 1 && c.width < (1u << 24), "width out of range");
  HCTR_CHECK(n_storage < 0x7fffffffull, "a shard holds fewer than 2^31 rows");
  HCTR_CHECK(root_arr != nullptr && (storage_arr != nullptr || n_storage == 0), "null root_arr / storage_arr");
  HCTR_CHECK(c.init_type >= 0 && c.init_type <= 3, "unknown initializer");

  kl.id_bits = std::max(1, bits_for(c.length - 1));
  kl.total_bits = kl.id_bits + (c.nrank > 1 ? bits_for((uint64_t)c.nrank - 1) : 0);
  HCTR_CHECK(kl.total_bits <= 64, "length * nrank does not fit a 64-bit sort key");
  kl.wide = kl.total_bits > 32;
  if (const char *f = getenv("HETUCTR_FORCE_WIDE_KEYS")) // exercises the 64-bit sort-key path on small tables
    if (f[0] == '1') kl.wide = true;
  // which sort indexes a batch: 0 the three-launch passes of radix_sort.h always, 2 the tile-sorted passes whenever
  // they can hold the batch (measurements of either sort at any size); default: tile_sort_fits()
  if (const char *f = getenv("HETUCTR_TILE_SORT")) tile_sort_mode = f[0] == '0' ? 0 : (f[0] == '2' ? 2 : 1);
  if (const char *f = getenv("HETUCTR_POOLED_FROM_KEYS")) pooled_from_keys = f[0] != '0';
  direct_gather_max = (uint32_t)std::min<uint64_t>(HCTR_DIRECT_GATHER_BYTES / ((uint64_t)c.width * sizeof(embed_t)), 0xfffffff0u);
  if (const char *f = getenv("HETUCTR_DIRECT_GATHER_MAX")) direct_gather_max = (uint32_t)strtoul(f, nullptr, 10);
  if (const char *f = getenv("HETUCTR_TILE_DIGIT_BITS")) // many narrow passes exercise the hand-over between the launches
    kl.max_digit_bits = atoi(f);

  // ---- host-side checks and the resident layout: cached ids first, then owned ids, order kept
  // (thrust::stable_partition at table_initialize.cu:81)
  const size_t L = c.length;
  size_t owned_total = 0;
  for (size_t i = 0; i < L; i++) {
    HCTR_CHECK(root_arr[i] < c.nrank, "root_arr holds an owner >= nrank");
    owned_total += root_arr[i] == c.rank;
  }
  std::vector<bool> seen(L, false);
  std::vector<index_t> ids(n_storage);
  size_t n_cached = 0, n_own = 0;
  for (size_t i = 0; i < n_storage; i++) {
    const int64_t id = storage_arr[i];
    HCTR_CHECK(id >= 0 && (uint64_t)id < L, "storage_arr holds an id outside [0, length)");
    HCTR_CHECK(!seen[id], "storage_arr holds an id twice");
    seen[id] = true;
    if (root_arr[id] != c.rank) ids[n_cached++] = id;
  }
  size_t w = n_cached;
  for (size_t i = 0; i < n_storage; i++)
    if (root_arr[storage_arr[i]] == c.rank) { ids[w++] = storage_arr[i]; n_own++; }
  // the reference only notices this when another shard queries the row (handle_query.cu:14-15)
  HCTR_CHECK(n_own == owned_total, "storage_arr must contain every id whose owner is this rank");
  n_owned = n_own;

  HCTR_HIP(hipSetDevice(cfg.device_id));
  hipStream_t s = group->stream;
  const size_t S = n_storage, C = n_cached, W = c.width;
  root.reserve(L);
  slot.reserve(L * sizeof(slot_t));
  store_ids.reserve(std::max<size_t>(S, 1) * sizeof(index_t));
  emb.reserve(std::max<size_t>(S * W, 1) * sizeof(embed_t));
  ver.reserve(std::max<size_t>(S, 1) * sizeof(version_t));
  pend.reserve(std::max<size_t>(C * W, 1) * sizeof(embed_t));
  upd.reserve(std::max<size_t>(C, 1) * sizeof(version_t));
  HCTR_HIP(hipMemcpyAsync(root.p, root_arr, L, hipMemcpyHostToDevice, s));
  if (S) HCTR_HIP(hipMemcpyAsync(store_ids.p, ids.data(), S * sizeof(index_t), hipMemcpyHostToDevice, s));
  launch_fill_i32(s, slot.as<int32_t>(), L, kNoSlot);
  launch_build_directory(s, store_ids.as<index_t>(), (uint32_t)S, slot.as<slot_t>());
  launch_init_values(s, emb.as<embed_t>(), S * W, c.init_type, c.init_a, c.init_b, seed);
  launch_fill_i64(s, ver.as<version_t>(), C, kInvalidVersion);          // table_initialize.cu:110
  launch_fill_i64(s, ver.as<version_t>() + C, S - C, 0);                // table_initialize.cu:111
  HCTR_HIP(hipMemsetAsync(pend.p, 0, pend.bytes, s));
  HCTR_HIP(hipMemsetAsync(upd.p, 0, upd.bytes, s));

  dstat.reserve(sizeof(DevStat));
  dst_ = dstat.as<DevStat>();
  stats.reserve(32);
  ret_seg_dev.reserve(2 * 258 * 4);
  HCTR_HIP(hipMemsetAsync(dstat.p, 0, dstat.bytes, s));
  HCTR_HIP(hipMemsetAsync(stats.p, 0, 32, s));
  for (Batch *b : {&cur, &prev}) {
    b->reserve(1, c.nrank, kl.wide);
    b->clear(s, c.nrank);
    b->send_cnt.assign(c.nrank + 1, 0);
    b->recv_cnt.assign(c.nrank + 1, 0);
    b->push_cnt.assign(c.nrank + 1, 0);
    b->pushrecv_cnt.assign(c.nrank + 1, 0);
  }
  rq_seg.assign(c.nrank + 1, 0);
  rg_seg.assign(c.nrank + 1, 0);
  ret_seg.assign(c.nrank + 1, 0);
  HCTR_HIP(hipHostMalloc((void **)&mirror, sizeof(HostMirror), hipHostMallocDefault));
  memset(mirror, 0, sizeof(HostMirror));
  HCTR_HIP(hipStreamSynchronize(s)); // root_arr / ids are host temporaries

  tv.rank = c.rank;
  tv.nrank = c.nrank;
  tv.id_max = L;
  tv.width = (uint32_t)W;
  tv.n_stored = (uint32_t)S;
  tv.n_cached = (uint32_t)C;
  tv.neg_lr = -c.learning_rate;
  tv.pull_bound = c.pull_bound;
  tv.push_bound = c.push_bound;
  tv.root = root.as<worker_t>();
  tv.slot = slot.as<slot_t>();
  tv.emb = emb.as<embed_t>();
  tv.ver = ver.as<version_t>();
  tv.pend = pend.as<embed_t>();
  tv.upd = upd.as<version_t>();
}

Shard::~Shard() {
  if (mirror) (void)hipHostFree(mirror);
}

void Shard::reserve_batch_scratch(uint32_t n) {
  const size_t m = std::max<uint32_t>(n, 1);
  const size_t ks = kl.wide ? 8 : 4;
  ktmp0.reserve(m * ks);
  ktmp1.reserve(m * ks);
  vtmp0.reserve(m * 4);
  vtmp1.reserve(m * 4);
  sortws.reserve(index_table_words(m) * 4);
  block_sums.reserve((scan_blocks(m) + 2) * 4);
  headws.reserve(head_chunk_words(m) * 4);
  sp.ktmp0 = ktmp0.p;
  sp.ktmp1 = ktmp1.p;
  sp.vtmp0 = vtmp0.as<uint32_t>();
  sp.vtmp1 = vtmp1.as<uint32_t>();
  sp.sortws = sortws.as<uint32_t>();
  sp.block_sums = block_sums.as<uint32_t>();
  sp.headws = headws.as<uint32_t>();
}

// the same pieces cut out of one caller-provided area (the static array) instead of the shard's own buffers, in the
// order and with the rounding of index_scratch_bytes
void Shard::use_scratch_area(void *area, uint32_t n) {
  const size_t m = std::max<uint32_t>(n, 1), ks = kl.wide ? 8 : 4;
  unsigned char *p = (unsigned char *)area;
  auto take = [&](size_t bytes) {
    void *r = p;
    p += index_scratch_round(bytes);
    return r;
  };
  sp.ktmp0 = take(m * ks);
  sp.ktmp1 = take(m * ks);
  sp.vtmp0 = (uint32_t *)take(m * 4);
  sp.vtmp1 = (uint32_t *)take(m * 4);
  sp.sortws = (uint32_t *)take(index_table_words(m) * 4);
  sp.block_sums = (uint32_t *)take((scan_blocks(m) + 2) * 4);
  sp.headws = (uint32_t *)take(head_chunk_words(m) * 4);
}

// csrc/core/preprocess.cu:92-141
void Shard::ingest_keys(const int64_t *keys, size_t n, uint32_t *flag, void *scratch_area) {
  HCTR_CHECK(n < 0xfffffff0ull, "a batch holds fewer than 2^32 keys");
  HCTR_CHECK(keys != nullptr || n == 0, "null key pointer");
  hipStream_t s = group->stream;
  cur.n = (uint32_t)n;
  cur.U = 0;
  cur.idx_map_valid = false;
  cur.planned = false;
  cur.lists_ready = n == 0;
  cur.direct_gather = false;
  cur.comp_valid = false;
  if (!scratch_area) cur.reserve(cur.n, cfg.nrank, kl.wide); // else: the caller has checked that the buffers hold n keys
  if (n == 0) { // :93-95
    cur.clear(s, cfg.nrank);
  } else {
    cur.cleared = false;
    u_cleared = false;
    if (scratch_area) use_scratch_area(scratch_area, cur.n);
    else reserve_batch_scratch(cur.n);
    {
      // ids -> device copy (:98-99) and sort keys.  When the caller's pointer is device-visible the copy is
      // written by the same kernel that reads the ids; a pageable host buffer goes through a transfer first.
      StageScope st(*group, S_KEYS);
      hipPointerAttribute_t attr;
      const bool visible = hipPointerGetAttributes(&attr, keys) == hipSuccess &&
                           (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged);
      bool narrowed = false;
      if (!visible) {
        (void)hipGetLastError(); // an unregistered host pointer leaves a sticky "invalid value"
        HCTR_CHECK(!scratch_area, "preprocess without allocations takes ids in device memory only (a transfer from "
                                  "pageable host memory needs a staging buffer)");
        // through pinned memory, as 32-bit ids when the table's ids fit (half the bytes on the bus)
        narrowed = tv.id_max <= 0xffffffffull;
        cur.staged.reserve(n * sizeof(index_t));
        stager.copy(cur.staged.p, keys, n * sizeof(index_t), s, narrowed);
      }
      const index_t *ids = visible ? (const index_t *)keys : (const index_t *)cur.staged.as<index_t>();
      cur.tile_sorted = tile_sort_mode == 2 ? tile_sort_possible(cur.n) : (tile_sort_mode == 1 && tile_sort_fits(cur.n));
      // A call that returns as soon as the ids are read (flag: where it looks for a bad id) gets them read by the
      // lightest kernel there is when the batch is large: the sort keys alone.  Sorting a tile as well keeps the
      // caller -- whose next call starts the gradient push -- waiting several microseconds longer.
      // One shard and a small batch: the step's gather works from the keys in batch order and leaves the index off
      // the step's critical path (write_back); the keys are then made by a kernel of their own here as well.
      cur.direct_gather = cfg.nrank == 1 && flag != nullptr && cur.n <= direct_gather_max;
      cur.keys_made = !cur.tile_sorted || (flag != nullptr && cur.n >= kKeysFirstFrom);
      cur.comp_valid = true; // either kernel leaves the sort keys in batch order (a gather from the keys reads them)
      if (!cur.keys_made)
        launch_tile_sort_keys(s, tv, kl, ids, nullptr, cur.n, tile_sort_buffers(), flag ? flag : err_ptr(),
                              cur.dnlong.as<uint32_t>(), narrowed, cur.comp.p);
      else
        launch_make_keys(s, tv, kl, ids, cur.n, cur.comp.p, flag ? flag : err_ptr(), cur.dnlong.as<uint32_t>(),
                         cur.tile_sorted ? nullptr : sp.sortws, narrowed);
    }
  }
}

TileSortBuffers Shard::tile_sort_buffers() const {
  TileSortBuffers b;
  b.keys[0] = sp.ktmp0;
  b.keys[1] = sp.ktmp1;
  b.vals[0] = sp.vtmp0;
  b.vals[1] = sp.vtmp1;
  b.tables = sp.sortws;
  return b;
}

void Shard::index_batch(uint32_t *u_out, int part) {
  hipStream_t s = group->stream;
  // part 1: the first launches of the sort; part 2: everything after them; 0: all of it
  if (cur.n != 0) {
    // head counts per chunk: one wave's share of a sort tile with the tile-sorted passes, else a tile of the unique pass
    const HeadChunks heads = head_chunks_in(sp.headws, cur.n, kl.wide, cur.tile_sorted ? (uint32_t)tile_items(cur.n) * kWave : 4096u);
    const void *sorted_keys = nullptr;
    {
      StageScope sort_scope(*group, S_SORT);
      if (cur.tile_sorted) {
        if (cur.keys_made && part != 2) // the sort's first launch, from the keys the call made before it returned
          launch_tile_sort_keys(s, tv, kl, nullptr, cur.comp.p, cur.n, tile_sort_buffers(), nullptr, nullptr);
        const int from = part == 2 ? 1 + kEarlyTilePasses : 1, to = part == 1 ? 1 + kEarlyTilePasses : (1 << 30);
        launch_tile_sort_passes(s, kl, cur.n, tile_sort_buffers(), cur.sorted_arg.as<uint32_t>(), heads, &sorted_keys,
                                from, to);
      } else {
        const int from = part == 2 ? kEarlySortSteps : 0, to = part == 1 ? kEarlySortSteps : (1 << 30);
        SortScratch sc;
        sc.words = sp.sortws;
        sc.n_cap = cur.n;
        if (kl.wide) {
          const uint64_t *sk;
          radix_sort_positions<uint64_t>(s, cur.comp.as<uint64_t>(), cur.n, kl.total_bits, (uint64_t *)sp.ktmp0,
                                         (uint64_t *)sp.ktmp1, sp.vtmp0, sp.vtmp1,
                                         cur.sorted_arg.as<uint32_t>(), sc, &sk, true, from, to);
          sorted_keys = sk;
        } else {
          const uint32_t *sk;
          radix_sort_positions<uint32_t>(s, cur.comp.as<uint32_t>(), cur.n, kl.total_bits, (uint32_t *)sp.ktmp0,
                                         (uint32_t *)sp.ktmp1, sp.vtmp0, sp.vtmp1,
                                         cur.sorted_arg.as<uint32_t>(), sc, &sk, true, from, to);
          sorted_keys = sk;
        }
      }
    }
    if (part == 1) return;
    StageScope st(*group, S_UNIQUE);
    launch_unique(s, tv, kl, sorted_keys, cur.view(), heads, !cur.tile_sorted, u_out ? u_out : &dst_->U);
    // the run lists follow in the gather of the step, or before the batch's push if that gather did not look at the
    // index or never came (lists_ready)
    // (built behind the index instead, they make the index the longer of a small step's two chains: 78 us against 64)
  }
  if (part == 1) return;
  if (cfg.nrank > 1) launch_bucket_sizes(s, cur.view(), cfg.nrank, dst_->send_cnt, mirror->st.send_cnt, &mirror->st.U);
}

// The push plan of a batch (csrc/core/preprocess.cu:148-182): which of its remote unique keys are pushed when it is
// the previous batch, and how many rows go to every owner.  It depends on the batch's index and on the update counters
// of the cached rows as the push of the step before left them, and nothing changes either between the end of that
// step and the preprocess call the reference computes the plan in: push_pull computes it for its current batch (beside
// the owner-side work, on the second stream), and the next preprocess finds it done.
void Shard::plan_batch(Batch &b) {
  hipStream_t s = group->stream;
  if (cfg.nrank == 1) return; // single shard: every key is owned, nothing is ever pushed
  if (b.n == 0) {
    for (int i = 0; i <= cfg.nrank; i++) mirror->st.push_cnt[i] = 0; // nothing in flight writes the block
    return;
  }
  b.need.reserve((size_t)b.n * 4);
  b.prefix.reserve((size_t)b.n * 4);
  b.plan_total.reserve(4);
  plan_sums.reserve((scan_blocks(b.n) + 2) * 4); // its own: the index of the next batch may be running beside it
  StageScope st(*group, S_PLAN);
  launch_decide_update(s, tv, kl, b.view(), b.need.as<uint32_t>());
  launch_exclusive_scan(s, b.need.as<uint32_t>(), b.prefix.as<uint32_t>(), b.n, b.dU.as<uint32_t>(),
                        plan_sums.as<uint32_t>(), b.plan_total.as<uint32_t>());
  launch_bucket_counts(s, b.view(), b.prefix.as<uint32_t>(), b.plan_total.as<uint32_t>(), cfg.nrank, dst_->push_cnt,
                       mirror->st.push_cnt);
}

void Shard::enqueue_readback_preprocess() {
  hipStream_t s = group->stream;
  if (cur.n == 0 && !u_cleared) {
    HCTR_HIP(hipMemsetAsync(&dst_->U, 0, 4, s));
    u_cleared = true;
  }
  // unique keys, error word, queries per owner; the pushed rows per owner reach the host from their own kernel
  const size_t bytes = cfg.nrank == 1 ? 16 : offsetof(DevStat, send_cnt) + (size_t)(cfg.nrank + 1) * sizeof(uint64_t);
  HCTR_HIP(hipMemcpyAsync(&mirror->st, dstat.p, bytes, hipMemcpyDeviceToHost, s));
}

void Shard::finish_preprocess() {
  if (!prev.planned) finish_plan(prev);
  finish_index();
}

// The two halves of what preprocess hands to the host, each written to the pinned block by the kernel that computes it:
// what the push plan of the previous batch produced (rows pushed per owner) and what the index of the current batch
// produced (unique keys, queries per owner).
void Shard::finish_plan(Batch &b) {
  if (cfg.nrank == 1) b.push_cnt[0] = 0;
  else
    for (int i = 0; i <= cfg.nrank; i++) b.push_cnt[i] = mirror->st.push_cnt[i];
  b.planned = true;
}

void Shard::finish_index() {
  cur.U = mirror->st.U;
  if (cfg.nrank == 1) cur.send_cnt[0] = cur.U;
  else
    for (int i = 0; i <= cfg.nrank; i++) cur.send_cnt[i] = mirror->st.send_cnt[i];
  check_key_error();
}

void Shard::check_key_error() {
  if (mirror->st.err) {
    const uint32_t e = mirror->st.err;
    mirror->st.err = 0;
    HCTR_HIP(hipMemsetAsync(err_ptr(), 0, 4, group->stream));
    HCTR_CHECK(!(e & 1u), "preprocess: a key lies outside [0, length) (it was treated as id 0)");
  }
}

// csrc/core/generate_query.cu:85-89; inference rule of csrc/core/hetu_gpu_table.cu:14-21
void Shard::begin_push(const float *grad, uint32_t bag) {
  hipStream_t s = group->stream;
  if (grad == nullptr) {
    prev.n = 0;
    prev.U = 0;
    prev.clear(s, cfg.nrank);
    std::fill(prev.push_cnt.begin(), prev.push_cnt.end(), 0);
    std::fill(prev.pushrecv_cnt.begin(), prev.pushrecv_cnt.end(), 0);
  }
  prev_active = prev.n > 0;
  last_stats[3] = 0;
  push_grad_ = grad;
  push_bag_ = bag;
  if (!prev_active) return;
  uint64_t pushes = 0;
  for (int i = 0; i < cfg.nrank; i++) pushes += prev.push_cnt[i];
  last_stats[3] = (long long)pushes;
  HCTR_CHECK(prev.n % bag == 0, "pooled push: the previous batch is not a whole number of bags");
}

void Shard::generate_gradient(const uint32_t *delta) {
  if (!prev_active) return;
  hipStream_t s = group->stream;
  PushArgs a;
  a.grad = push_grad_;
  a.bag = BagDiv(push_bag_);
  a.need = nullptr;
  a.prefix = nullptr;
  a.g_idx = nullptr;
  a.g_cnt = nullptr;
  a.g_val = nullptr;
  if (!prev.lists_ready) { // no gather has seen this batch (a second preprocess came first, or a call without output)
    launch_list_long_runs(s, prev.view());
    prev.lists_ready = true;
  }
  StageScope st(*group, S_PUSH);
  if (cfg.nrank > 1) {
    // the pushed rows go straight into the group's receive area: plan position -> position there
    push_pos.reserve((size_t)std::max<uint32_t>(prev.U, 1) * 4);
    launch_place_rows(s, kl, prev.view(), prev.U, prev.prefix.as<uint32_t>(), delta, push_pos.as<uint32_t>());
    a.need = prev.need.as<uint32_t>();
    a.prefix = push_pos.as<uint32_t>();
    a.g_idx = group->rg_idx_all.as<index_t>();
    a.g_cnt = group->rg_cnt_all.as<version_t>();
    a.g_val = group->rg_val_all.as<embed_t>();
  }
  launch_push(s, tv, kl, prev.view(), prev.U, a);
}

// csrc/core/generate_query.cu:91-106
void Shard::generate_query(const uint32_t *delta) {
  if (cfg.nrank == 1) return; // a shard never finds its own rows outdated (handle_query.cu:47-54)
  hipStream_t s = group->stream;
  StageScope st(*group, S_QUERY);
  // every query is written where its owner reads it: the group's receive area (see Group::place_queries)
  launch_build_queries(s, tv, kl, cur.view(), cur.n, delta, group->rq_idx_all.as<index_t>(),
                       group->rq_ver_all.as<version_t>());
}

// What the owner-side kernels need of this shard for the step (csrc/core/handle_query.cu:7-116): the received pushes
// and queries, the buffers of the rows that go back.  The number of rows that go back to every requester stays on the
// device, where the owners' kernels read it; the host copy (statistics, error flags) is written by the same kernel
// into pinned memory and read when the step is over.
void Shard::fill_owner_args(OwnerShard &o, uint64_t queries_max) {
  const int R = cfg.nrank;
  query_sums.reserve((query_tiles((uint32_t)queries_max) + 2) * 4);
  // requester role: what comes back lands here (a row per unique key at most, and the host has not seen how many of
  // the batch's keys are unique), written by the owners
  const size_t rows_ub = std::max<uint32_t>(cur.n, 1);
  got.reserve(rows_ub * 4);
  in_ver.reserve(rows_ub * sizeof(version_t));
  in_val.reserve(rows_ub * cfg.width * sizeof(embed_t));
  last_stats[5] = (long long)rg_seg[R];
  o.t = tv;
  o.rg_idx = group->rg_idx_all.as<index_t>() + rg_base;
  o.rg_cnt = group->rg_cnt_all.as<version_t>() + rg_base;
  o.rg_val = group->rg_val_all.as<embed_t>() + rg_base * cfg.width;
  o.longest = 0;
  for (int i = 0; i <= R; i++) o.rg_seg[i] = (uint32_t)rg_seg[i];
  for (int i = 1; i < R; i++)
    if (rg_seg[i + 1] - rg_seg[i] > rg_seg[o.longest + 1] - rg_seg[o.longest]) o.longest = i;
  o.push_blocks = div_up(rg_seg[o.longest + 1] - rg_seg[o.longest], owner_push_rows_per_block(tv.width));
  // the received queries: place_queries fills in where they lie and how many they are (rq_idx .. got_delta)
  o.send_cnt = dst_->send_cnt;
  o.n_keys = cur.n;
  o.rq_idx = nullptr;
  o.rq_ver = nullptr;
  o.q = 0;
  o.query_tiles = 1;
  o.outdated = nullptr;
  o.ret_slot = nullptr;
  o.q_slot = nullptr;
  o.tile_cnt = query_sums.as<uint32_t>();
  o.in_ver = in_ver.as<version_t>();
  o.in_val = in_val.as<embed_t>();
  o.ret_delta = group->ret_delta_dev.as<uint32_t>() + (size_t)cfg.rank * R;
  o.got = got.as<uint32_t>();
  o.err = err_ptr();
  o.seg_dev = ret_seg_dev.as<uint32_t>();
  o.seg_host = mirror->ret_seg;
}

void Shard::finish_handle_query() {
  for (int i = 0; i <= cfg.nrank; i++) ret_seg[i] = mirror->ret_seg[i];
  last_stats[4] = (long long)ret_seg[cfg.nrank];
  if (mirror->ret_seg[257]) {
    const uint32_t e = mirror->ret_seg[257];
    HCTR_HIP(hipMemsetAsync(err_ptr(), 0, 4, group->stream));
    HCTR_CHECK(!(e & 2u), "a pushed row reached a shard that does not own it");
    HCTR_CHECK(!(e & 4u), "a queried row reached a shard that does not own it");
  }
}

// whether this step's gather works from the keys in batch order (and the step does not wait for the index)
// (bags: a pooled gather walks the batch in its own order anyway, so it always works from the keys when they are there)
bool Shard::direct_now(uint32_t bag) const {
  if (cfg.nrank != 1 || !cur.comp_valid || cur.n == 0) return false;
  return bag == 1 ? cur.direct_gather : pooled_from_keys;
}

// csrc/core/writeback.cu:43-56
void Shard::write_back(float *dst, uint32_t bag) {
  hipStream_t s = group->stream;
  PullArgs a;
  a.got = nullptr;
  a.ret_i = nullptr;
  a.src_row = nullptr;
  a.in_ver = nullptr;
  a.in_val = nullptr;
  a.dst = dst;
  a.list_chunks = 0;
  // The gathered rows are not read again by this library: streamed past the caches they leave the table rows of the
  // batch there for the push that updates them next.  The one case where that loses is a batch of (almost) all
  // distinct keys, where the gather reads as many rows as it writes; the previous batch is the predictor.
  a.stream_stores = !(prev.n != 0 && (double)prev.U >= 0.9 * (double)prev.n);
  if (cfg.nrank > 1 && cur.n == 0) {
    memset(mirror->stats, 0, sizeof mirror->stats); // no keys: nothing came back (nothing in flight writes the block)
  } else if (cfg.nrank > 1) {
    // sized for the batch's keys: how many of them are unique the kernels read on the device (the host has not
    // waited for the index); the scan scratch is the one the batch's index was given, its kernels are through
    ret_i.reserve((size_t)cur.n * 4);
    src_row.reserve((size_t)cur.n * 4);
    StageScope st(*group, S_REFRESH);
    a.got = got.as<uint32_t>();
    a.ret_i = ret_i.as<uint32_t>();
    a.src_row = src_row.as<uint32_t>();
    a.in_ver = in_ver.as<version_t>();
    a.in_val = in_val.as<embed_t>();
    launch_refresh(s, tv, cur.view(), cur.n, prev.U ? prev.U : cur.n, a, sp.block_sums, stats.as<uint32_t>(), mirror->stats);
  }
  if (dst != nullptr && direct_now(bag)) {
    StageScope st(*group, S_GATHER);
    HCTR_CHECK(cur.n % bag == 0, "pooled pull: the batch is not a whole number of bags");
    if (bag > 1) launch_gather_pooled_direct(s, tv, kl, cur.comp.p, cur.n, dst, bag);
    else launch_gather_direct(s, tv, kl, cur.comp.p, cur.n, dst, a.stream_stores);
  } else if (dst != nullptr) {
    StageScope st(*group, S_GATHER);
    if (!cur.lists_ready && cur.n != 0) { // the first blocks of the gather build the batch's run lists on their way
      a.list_chunks = run_list_chunks(cur.n);
      cur.lists_ready = true;
    }
    if (bag > 1) { // sum-pooled bags: in batch order, through the inverse index
      HCTR_CHECK(cur.n % bag == 0, "pooled pull: the batch is not a whole number of bags");
      if (!cur.idx_map_valid) {
        launch_idx_map(s, cur.view());
        cur.idx_map_valid = true;
      }
      launch_gather_pooled(s, tv, cur.view(), a, bag);
    } else {
      launch_gather(s, tv, cur.view(), a);
    }
  }
}

void Shard::finish_push_pull() {
  if (cfg.nrank > 1) {
    last_stats[0] = mirror->stats[0];
    last_stats[1] = mirror->stats[1];
    last_stats[2] = mirror->stats[2];
    HCTR_CHECK(!(mirror->stats[3] & 8u), "an owned row came back as outdated");
  }
}

// ---- introspection -------------------------------------------------------------------------------
namespace {
template <typename T> std::vector<T> download(const void *dev, size_t n) {
  std::vector<T> h(n);
  if (n) HCTR_HIP(hipMemcpy(h.data(), dev, n * sizeof(T), hipMemcpyDeviceToHost));
  return h;
}
template <typename V> size_t put64(const V &v, size_t n, void *out, size_t cap) {
  long long *o = (long long *)out;
  for (size_t i = 0; i < n && i < cap; i++) o[i] = (long long)v[i];
  return n;
}
} // namespace

size_t Shard::fetch(int which, void *out, size_t cap) {
  HCTR_HIP(hipSetDevice(cfg.device_id));
  group->flush_index();
  HCTR_HIP(hipStreamSynchronize(group->stream));
  const int R = cfg.nrank;
  const uint64_t id_mask = kl.id_bits >= 64 ? ~0ull : (((uint64_t)1 << kl.id_bits) - 1);
  auto ukeys = [&](const Batch &b) {
    std::vector<uint64_t> k(b.U);
    if (kl.wide) {
      auto h = download<uint64_t>(b.ukey.p, b.U);
      for (size_t i = 0; i < b.U; i++) k[i] = h[i];
    } else {
      auto h = download<uint32_t>(b.ukey.p, b.U);
      for (size_t i = 0; i < b.U; i++) k[i] = h[i];
    }
    return k;
  };
  switch (which) {
    case HCTR_F_UNIQUE: { auto k = ukeys(cur); for (auto &x : k) x &= id_mask; return put64(k, cur.U, out, cap); }
    case HCTR_F_ROOT: { auto k = ukeys(cur); for (auto &x : k) x >>= kl.id_bits; return put64(k, cur.U, out, cap); }
    case HCTR_F_SORTED_ARG: return put64(download<uint32_t>(cur.sorted_arg.p, cur.n), cur.n, out, cap);
    case HCTR_F_RUN_START: return put64(download<uint32_t>(cur.run_start.p, (size_t)cur.U + 1), (size_t)cur.U + 1, out, cap);
    case HCTR_F_IDX_MAP: {
      if (!cur.idx_map_valid) {
        launch_idx_map(group->stream, cur.view());
        HCTR_HIP(hipStreamSynchronize(group->stream));
        cur.idx_map_valid = true;
      }
      return put64(download<uint32_t>(cur.idx_map.p, cur.n), cur.n, out, cap);
    }
    case HCTR_F_OFFSET: return put64(download<slot_t>(cur.uoff.p, cur.U), cur.U, out, cap);
    case HCTR_F_SEND_CNT: return put64(cur.send_cnt, R, out, cap);
    case HCTR_F_RECV_CNT: return put64(cur.recv_cnt, R, out, cap);
    case HCTR_F_NEED_UPDATE:
    case HCTR_F_UPDATE_PREFIX: {
      if (R == 1 || prev.U == 0) { std::vector<long long> z(prev.U, 0); return put64(z, prev.U, out, cap); }
      return put64(download<uint32_t>(which == HCTR_F_NEED_UPDATE ? prev.need.p : prev.prefix.p, prev.U), prev.U, out, cap);
    }
    case HCTR_F_PUSH_CNT: return put64(prev.push_cnt, R, out, cap);
    case HCTR_F_PUSHRECV_CNT: return put64(prev.pushrecv_cnt, R, out, cap);
    case HCTR_F_OUTDATED: {
      if (R == 1) { std::vector<long long> z(cur.U, 0); return put64(z, cur.U, out, cap); }
      return put64(download<uint32_t>(group->rq_outdated_all.as<uint32_t>() + rq_base, rq_seg[R]), rq_seg[R], out, cap);
    }
    case HCTR_F_GOT: {
      if (R == 1) { std::vector<long long> z(cur.U, 0); return put64(z, cur.U, out, cap); }
      return put64(download<uint32_t>(got.p, cur.U), cur.U, out, cap);
    }
    case HCTR_F_VERSION: return put64(download<version_t>(ver.p, tv.n_stored), tv.n_stored, out, cap);
    case HCTR_F_UPDATES: return put64(download<version_t>(upd.p, tv.n_cached), tv.n_cached, out, cap);
    case HCTR_F_STORE_IDS: return put64(download<index_t>(store_ids.p, tv.n_stored), tv.n_stored, out, cap);
    case HCTR_F_KEYS: { // the ids of the batch as its sort keys hold them (an id outside the table reads as 0)
      std::vector<uint64_t> k(cur.n);
      if (!cur.comp_valid) { // no copy in batch order was kept: position sorted_arg[j] holds the key of rank_sorted[j]
        const auto uk = ukeys(cur);
        const auto pos = download<uint32_t>(cur.sorted_arg.p, cur.n), rk = download<uint32_t>(cur.rank_sorted.p, cur.n);
        for (size_t j = 0; j < cur.n; j++) k[pos[j]] = uk[rk[j]] & id_mask;
      } else if (kl.wide) {
        auto h = download<uint64_t>(cur.comp.p, cur.n);
        for (size_t i = 0; i < cur.n; i++) k[i] = h[i] & id_mask;
      } else {
        auto h = download<uint32_t>(cur.comp.p, cur.n);
        for (size_t i = 0; i < cur.n; i++) k[i] = h[i] & id_mask;
      }
      return put64(k, cur.n, out, cap);
    }
    case HCTR_F_EMBEDDING:
    case HCTR_F_PENDING: {
      const size_t n = (size_t)(which == HCTR_F_EMBEDDING ? tv.n_stored : tv.n_cached) * tv.width;
      const void *src = which == HCTR_F_EMBEDDING ? emb.p : pend.p;
      if (std::min(n, cap)) HCTR_HIP(hipMemcpy(out, src, std::min(n, cap) * sizeof(embed_t), hipMemcpyDeviceToHost));
      return n;
    }
    case HCTR_F_STATS: return put64(last_stats, 6, out, cap);
    case HCTR_F_SIZES: {
      long long z[6] = {(long long)cur.n, (long long)cur.U, (long long)prev.n, (long long)prev.U,
                        (long long)tv.n_stored, (long long)tv.n_cached};
      return put64(z, 6, out, cap);
    }
  }
  throw Error("hetuCTR: unknown item for debug_fetch");
}

// ================================================================================================
// Group
// ================================================================================================
Group::Group(int nr, int dev, std::string k) : nrank(nr), device_id(dev), key(std::move(k)), members(nr, nullptr) {
  int ndev = 0;
  HCTR_HIP(hipGetDeviceCount(&ndev));
  HCTR_CHECK(dev >= 0 && dev < ndev, "InCorrect device number."); // table_initialize.cu:144-146
  HCTR_HIP(hipSetDevice(dev));
  noalloc_scratch = noalloc_scratch_of(dev); // this device's copy of the static array, looked up with it current
  // a blocking stream, like the reference's cudaStreamCreate (table_initialize.cu:16): work the caller queued on the
  // legacy default stream (torch's default) is ordered before ours without an explicit synchronisation
  HCTR_HIP(hipStreamCreate(&stream));
  HCTR_HIP(hipStreamCreate(&index_stream));
  HCTR_HIP(hipEventCreateWithFlags(&ev_index, hipEventDisableTiming));
  HCTR_HIP(hipEventCreateWithFlags(&ev_keys, hipEventDisableTiming));
  HCTR_HIP(hipEventCreate(&ev_push));
  HCTR_HIP(hipEventCreateWithFlags(&ev_pushed, hipEventDisableTiming));
  HCTR_HIP(hipEventCreateWithFlags(&ev_plan, hipEventDisableTiming));
  const char *defer = getenv("HETUCTR_DEFER_INDEX");
  defer_index = !(defer && atoi(defer) == 0);
  HCTR_HIP(hipEventCreate(&ev0));
  HCTR_HIP(hipEventCreate(&ev1));
  a_keys_.resize(nr);
  a_n_.resize(nr);
  a_grad_.resize(nr);
  a_dst_.resize(nr);
  a_bag_.resize(nr, 1);
  if (const char *w = getenv("HETUCTR_GROUP_WAIT_SECONDS")) wait_seconds = atof(w);
}

Group::~Group() {
  if (ev0) (void)hipEventDestroy(ev0);
  if (ev1) (void)hipEventDestroy(ev1);
  for (auto &m : marks) { (void)hipEventDestroy(m.a); (void)hipEventDestroy(m.b); }
  for (auto e : event_pool) (void)hipEventDestroy(e);
  if (stream) (void)hipStreamDestroy(stream);
  if (index_stream) (void)hipStreamDestroy(index_stream);
  if (ev_index) (void)hipEventDestroy(ev_index);
  if (ev_keys) (void)hipEventDestroy(ev_keys);
  if (ev_push) (void)hipEventDestroy(ev_push);
  if (ev_pushed) (void)hipEventDestroy(ev_pushed);
  if (ev_plan) (void)hipEventDestroy(ev_plan);
  if (owner_host) (void)hipHostFree(owner_host);
  if (push_delta_host) (void)hipHostFree(push_delta_host);
}

void Group::join(Shard *s) {
  std::lock_guard<std::mutex> lk(mu_);
  HCTR_CHECK(members[s->cfg.rank] == nullptr, "this rank already exists in the group named by (ip, port)");
  members[s->cfg.rank] = s;
}

void Group::leave(Shard *s) {
  std::lock_guard<std::mutex> lk(mu_);
  // The shard's buffers are about to be freed: nothing of it may still be running, and what a deferred preprocess
  // left behind is taken over while every member is still there (the survivors of a group keep the sizes of their
  // current batches; the group itself cannot step again without the rank that leaves).
  if (index_pending || index_rest_pending) {
    try {
      if (complete()) flush_index();
    } catch (const std::exception &) {
      // a bad key of the abandoned batch: nobody is left to report it to
    }
    index_pending = false;
    index_rest_pending = false;
    (void)hipStreamSynchronize(index_stream);
  }
  if (members[s->cfg.rank] == s) members[s->cfg.rank] = nullptr;
}

bool Group::complete() const {
  for (Shard *m : members)
    if (!m) return false;
  return true;
}

hipEvent_t Group::take_event() {
  if (!event_pool.empty()) {
    hipEvent_t e = event_pool.back();
    event_pool.pop_back();
    return e;
  }
  hipEvent_t e;
  HCTR_HIP(hipEventCreate(&e));
  return e;
}

void Group::collect_marks() {
  for (auto &m : marks) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, m.a, m.b) == hipSuccess) {
      stage_ms[m.stage] += ms;
      stage_calls[m.stage]++;
    }
    event_pool.push_back(m.a);
    event_pool.push_back(m.b);
  }
  marks.clear();
}

// handleGradient + handleQuery of every shard (csrc/core/hetu_gpu_table.cu:27-31): one set of launches for the group
void Group::owner_side(uint64_t queries_max) {
  uint32_t push_blocks = 0;
  for (int r = 0; r < nrank; r++) push_blocks = std::max(push_blocks, owner_host[r].push_blocks);
  StageScope st(*this, S_OWNER);
  // the grids of the query kernels: from what the busiest owner received in the step before (the first step: the most)
  const uint32_t guess = queries_seen_ ? queries_guess_ : (uint32_t)queries_max;
  launch_owner_side(stream, owner_dev.as<OwnerShard>(), nrank, nrank, members[0]->cfg.width, push_blocks, (uint32_t)queries_max,
                    guess);
}

void Group::set_defer_index(bool on) {
  std::lock_guard<std::mutex> lk(mu_);
  flush_index();
  defer_index = on;
}

void Group::set_call_timing(bool on) {
  std::lock_guard<std::mutex> lk(mu_);
  time_calls = on;
  for (Shard *m : members)
    if (m) m->last_pre_ms = m->last_pp_ms = m->last_push_ms = 0.f;
}

void Group::set_stage_timing(bool on) {
  std::lock_guard<std::mutex> lk(mu_); // not while the ranks of the group are inside a collective call
  flush_index();
  stage_timing = on;
  for (int i = 0; i < S_COUNT; i++) {
    stage_ms[i] = 0;
    stage_calls[i] = 0;
  }
}

// The pushes of a step never pass through a send buffer: a pushed row is written by the push kernel into the receive
// area of its owner (csrc/core/all2all.cu:48-87 moves it there in the reference).  How many rows every shard pushes to
// every owner is known from the plans before any push kernel starts, so the area is sized and cut here: one piece per
// owner, inside it one per source, both in rank order.  In one process the area is one allocation; between GPUs every
// owner would hold its piece and hand its address to the others.
void Group::place_pushes() {
  const int R = nrank;
  if (R == 1) return;
  if (!push_delta_host) {
    HCTR_HIP(hipHostMalloc((void **)&push_delta_host, (size_t)R * R * sizeof(uint32_t), hipHostMallocDefault));
    push_delta_dev.reserve((size_t)R * R * sizeof(uint32_t));
  }
  uint64_t total = 0;
  for (int d = 0; d < R; d++) {
    Shard &dst = *members[d];
    dst.rg_base = total;
    uint64_t G = 0;
    for (int s = 0; s < R; s++) {
      dst.rg_seg[s] = G;
      if (members[s]->prev_active) G += members[s]->prev.push_cnt[d];
    }
    dst.rg_seg[R] = G;
    total += G;
  }
  HCTR_CHECK(total < 0xfffffff0ull, "more than 2^32 rows are pushed in one step");
  if (!total) return;
  const size_t W = members[0]->cfg.width;
  rg_idx_all.reserve(total * sizeof(index_t));
  rg_cnt_all.reserve(total * sizeof(version_t));
  rg_val_all.reserve(total * W * sizeof(embed_t));
  for (int s = 0; s < R; s++) {
    Shard &src = *members[s];
    uint64_t glo = 0; // rows of this source for the owners before d
    for (int d = 0; d < R; d++) {
      const Shard &dst = *members[d];
      // (place in the area) - (place in the source's plan), modulo 2^32 like the sum the kernel forms
      push_delta_host[(size_t)s * R + d] = (uint32_t)(dst.rg_base + dst.rg_seg[s] - glo);
      if (src.prev_active) glo += src.prev.push_cnt[d];
    }
  }
  HCTR_HIP(hipMemcpyAsync(push_delta_dev.p, push_delta_host, (size_t)R * R * sizeof(uint32_t), hipMemcpyHostToDevice, stream));
}

// csrc/core/all2all.cu:18-46: every owner's receive buffer is the requesters' buckets for it, in source order.  The
// queries do not pass through a send buffer either: every shard's query kernel writes into one receive area of the
// group, cut into one piece per owner and, inside it, one per source; a unique key of rank u lands u + (distance for its
// owner) into the area.  How many unique keys every shard asks every owner for is left on the device by the shards'
// index kernels, and the host does not wait for them: the area is sized here for the most queries there can be (a batch
// has no more unique keys than keys) and cut on the device (launch_place_queries), which also tells every owner where
// its piece lies.  Returns that maximum.
uint64_t Group::reserve_queries() {
  const int R = nrank;
  if (R == 1) return 0;
  uint64_t most = 0;
  for (Shard *m : members) most += m->cur.n;
  HCTR_CHECK(most < 0xfffffff0ull, "more than 2^32 queries in one step");
  const uint64_t cap = std::max<uint64_t>(most, 1);
  rq_idx_all.reserve(cap * sizeof(index_t));
  rq_ver_all.reserve(cap * sizeof(version_t));
  rq_outdated_all.reserve(cap * 4);
  rq_slot_all.reserve(cap * sizeof(slot_t));
  rq_ret_all.reserve(cap * sizeof(slot_t));
  query_delta_dev.reserve((size_t)R * R * sizeof(uint32_t));
  return most;
}

QueryArea Group::query_area() {
  QueryArea a;
  a.idx = rq_idx_all.as<index_t>();
  a.ver = rq_ver_all.as<version_t>();
  a.outdated = rq_outdated_all.as<uint32_t>();
  a.q_slot = rq_slot_all.as<slot_t>();
  a.ret_slot = rq_ret_all.as<slot_t>();
  a.query_delta = query_delta_dev.as<uint32_t>();
  return a;
}

// what launch_place_queries computed, once more on the host when the step is over (introspection reads it)
void Group::note_query_places() {
  const int R = nrank;
  uint64_t total = 0, busiest = 0;
  for (int d = 0; d < R; d++) {
    Shard &dst = *members[d];
    dst.rq_base = total;
    uint64_t Q = 0;
    for (int s = 0; s < R; s++) {
      dst.rq_seg[s] = Q;
      Q += members[s]->cur.send_cnt[d];
    }
    dst.rq_seg[R] = Q;
    total += Q;
    busiest = std::max(busiest, Q);
  }
  queries_guess_ = (uint32_t)busiest;
  queries_seen_ = true;
}

// csrc/core/hetu_gpu_table.cu:43-65 for every shard of the group
// Waits for the stream by polling: the calls are short and a blocking wait adds tens of microseconds of
// wake-up latency to each of them.
void Group::sync_stream() { HCTR_HIP(hipStreamSynchronize(stream)); }

namespace {
void wait_for(hipStream_t s) { HCTR_HIP(hipStreamSynchronize(s)); }
} // namespace

// Enqueues index stages of the ingested batch (single shard) on the stream the stages currently use.
// The number of unique keys is written by its kernel straight into the pinned host block finish_preprocess() reads: no
// copy stands between the last index kernel and the gather that waits for it.
static void enqueue_index(Shard *m, int part) {
  if (m->cur.n == 0) m->mirror->st.U = 0; // nothing of this shard is in flight that writes the block
  m->index_batch(&m->mirror->st.U, part);
}

// several shards: one part of the index of every shard's current batch, on the second stream
void Group::enqueue_index_all(int part) {
  StreamSwitch on(*this, index_stream);
  for (Shard *m : members) {
    if (m->cur.n == 0) { // an empty batch (a shard that only serves): nothing to launch, nothing to read back
      m->mirror->st.U = 0;
      for (int i = 0; i <= nrank; i++) m->mirror->st.send_cnt[i] = 0;
      continue;
    }
    m->index_batch(nullptr, part);
  }
}

// the launches of the index that preprocess left to the next call
void Group::enqueue_index_rest() {
  if (!index_rest_pending) return;
  index_rest_pending = false;
  if (nrank == 1) {
    StreamSwitch on(*this, index_stream);
    enqueue_index(members[0], 2);
    HCTR_HIP(hipEventRecord(ev_index, stream));
  } else {
    enqueue_index_all(2);
  }
  index_pending = true;
}

void Group::flush_index() {
  if (!index_pending && !index_rest_pending) return;
  HCTR_HIP(hipSetDevice(device_id));
  enqueue_index_rest();
  index_pending = false;
  wait_for(index_stream);
  if (nrank == 1) members[0]->finish_preprocess();
  else
    for (Shard *m : members) m->finish_index(); // the plan half was taken over when preprocess returned
  exchange_shapes();
}

void Group::preprocess_all(const int64_t *const *keys, const size_t *n) {
  HCTR_CHECK(complete(), "the loopback group named by (ip, port) is missing ranks");
  HCTR_HIP(hipSetDevice(device_id));
  flush_index(); // preprocess twice in a row: the earlier batch is indexed before it becomes the previous one
  if (defer_index && !stage_timing && nrank == 1) {
    // One shard: everything is enqueued on the second stream, and the call returns as soon as the caller's ids have
    // been read.  Sorting and deduplicating them does not depend on the pending gradient push, which the next
    // push_pull puts on the main stream while this is still running; the gather waits for both.
    // The host returns as early as it can, because the caller's next call is what starts the gradient push: only
    // the first launches of the index are enqueued here (they keep the GPU busy until that push arrives), the rest
    // follows from push_pull once the push kernel is in its queue.
    Shard *m = members[0];
    StreamSwitch on(*this, index_stream);
    if (time_calls) HCTR_HIP(hipEventRecord(ev0, stream));
    m->swap_batches();
    m->ingest_keys(keys[0], n[0], &m->mirror->key_err); // the flag lives in pinned host memory the kernel can write
    if (time_calls) HCTR_HIP(hipEventRecord(ev1, stream));
    HCTR_HIP(hipEventRecord(ev_keys, stream));
    enqueue_index(m, 1);
    index_rest_pending = true;
    HCTR_HIP(hipEventSynchronize(ev_keys));
    if (time_calls) {
      float ms = 0.f;
      HCTR_HIP(hipEventElapsedTime(&ms, ev0, ev1));
      m->last_pre_ms = ms;
    }
    if (m->mirror->key_err) {
      m->mirror->key_err = 0;
      throw Error("hetuCTR: preprocess: a key lies outside [0, length) (it was treated as id 0)");
    }
    return;
  }
  if (defer_index && !stage_timing) {
    // Several shards: as with one, the ids are read by a kernel on the second stream and the call returns when that
    // kernel is through; the index of the current batches follows on that stream (no event between the two streams:
    // waiting for one costs the host 15-20 us), next to the pushes that the next push_pull queues first.  push_pull
    // waits for the index before it builds the queries, which are the first thing that needs it.  The push plan of the
    // previous batches was made at the end of the step before.
    std::vector<Shard *> late;
    for (Shard *m : members) m->swap_batches();
    // a previous batch that no push_pull has seen yet (two preprocess calls in a row) is planned here, on the main
    // stream, and waited for (the plan sizes the push buffers)
    for (Shard *m : members)
      if (!m->prev.planned) {
        m->plan_batch(m->prev);
        late.push_back(m);
      }
    {
      StreamSwitch on(*this, index_stream);
      if (time_calls) HCTR_HIP(hipEventRecord(ev0, stream));
      for (Shard *m : members) m->ingest_keys(keys[m->cfg.rank], n[m->cfg.rank], &m->mirror->key_err);
      if (time_calls) HCTR_HIP(hipEventRecord(ev1, stream));
      HCTR_HIP(hipEventRecord(ev_keys, stream));
    }
    // Only the first launches of the index go out here (they keep the GPU busy until the pushes arrive); the rest
    // follows from push_pull once the push kernels are in their queue.
    enqueue_index_all(1);
    index_rest_pending = true;
    HCTR_HIP(hipEventSynchronize(ev_keys)); // the ids have been read: the caller may reuse its buffers
    if (!late.empty()) sync_stream();
    for (Shard *m : late) m->finish_plan(m->prev);
    float ms = 0.f;
    if (time_calls) HCTR_HIP(hipEventElapsedTime(&ms, ev0, ev1));
    bool bad_key = false;
    for (Shard *m : members) {
      m->last_pre_ms = ms;
      bad_key |= m->mirror->key_err != 0;
      m->mirror->key_err = 0;
    }
    exchange_shapes();
    if (bad_key) throw Error("hetuCTR: preprocess: a key lies outside [0, length) (it was treated as id 0)");
    return;
  }
  if (time_calls) HCTR_HIP(hipEventRecord(ev0, stream));
  for (Shard *m : members) {
    m->swap_batches();
    m->preprocess_index(keys[m->cfg.rank], n[m->cfg.rank]);
    if (!m->prev.planned) m->plan_batch(m->prev);
    m->enqueue_readback_preprocess();
  }
  if (time_calls) HCTR_HIP(hipEventRecord(ev1, stream));
  sync_stream();
  float ms = 0.f;
  if (time_calls) HCTR_HIP(hipEventElapsedTime(&ms, ev0, ev1));
  collect_marks();
  std::string first_error;
  for (Shard *m : members) {
    m->last_pre_ms = ms;
    try {
      m->finish_preprocess();
    } catch (const Error &e) {
      if (first_error.empty()) first_error = e.what();
    }
  }
  exchange_shapes();
  if (!first_error.empty()) throw Error(first_error);
}

// hctr_preprocess_noalloc: the literal contract of HetuTable::preprocess (everything done when the call returns) for one
// shard, with every piece of index scratch taken from the static array and no allocation anywhere on the way.
void Group::preprocess_noalloc(const int64_t *keys, size_t n) {
  HCTR_CHECK(nrank == 1, "preprocess without allocations is built for a table of one shard");
  HCTR_CHECK(n <= kNoAllocMaxKeys, "preprocess without allocations takes at most " + std::to_string(kNoAllocMaxKeys) +
                                       " keys per batch (the size of its static scratch)");
  HCTR_CHECK(!stage_timing, "stage timing takes events from a growing pool: switch it off for calls that may not allocate");
  HCTR_HIP(hipSetDevice(device_id));
  flush_index(); // an earlier deferred batch is indexed before it becomes the previous one
  Shard *m = members[0];
  // after the swap the current batch lives in the buffers of the batch before the previous one
  HCTR_CHECK(m->prev.holds((uint32_t)n, 1, m->kl.wide),
             "preprocess without allocations: the table's batch buffers are smaller than this batch; they are sized by "
             "ordinary hctr_preprocess calls (two in a row size both)");
  HCTR_CHECK(index_scratch_bytes((uint32_t)n, m->kl.wide) <= kNoAllocScratchBytes, "internal: static scratch too small");
  if (n) {
    hipPointerAttribute_t attr;
    const bool visible = keys != nullptr && hipPointerGetAttributes(&attr, keys) == hipSuccess &&
                         (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged);
    if (!visible) (void)hipGetLastError();
    HCTR_CHECK(visible, "preprocess without allocations takes ids in device memory only (a transfer from pageable "
                        "host memory needs a staging buffer)");
  }
  m->swap_batches();
  m->ingest_keys(keys, n, nullptr, noalloc_scratch);
  m->index_batch();
  m->enqueue_readback_preprocess();
  sync_stream();
  m->finish_preprocess();
  exchange_shapes();
}

// all2allExchangeShape, csrc/core/all2all.cu:6-16
void Group::exchange_shapes() {
  for (Shard *m : members)
    for (int s = 0; s < nrank; s++) {
      m->cur.recv_cnt[s] = members[s]->cur.send_cnt[m->cfg.rank];
      m->prev.pushrecv_cnt[s] = members[s]->prev.push_cnt[m->cfg.rank];
    }
}

// csrc/core/hetu_gpu_table.cu:9-41 for every shard of the group
void Group::push_pull_all(const float *const *grads, float *const *dsts, size_t bag_size) {
  HCTR_CHECK(bag_size >= 1 && bag_size < (1u << 24), "bag size out of range");
  const uint32_t bag = (uint32_t)bag_size;
  HCTR_CHECK(complete(), "the loopback group named by (ip, port) is missing ranks");
  HCTR_HIP(hipSetDevice(device_id));
  // every caller error that can be seen from the arguments is reported here, before any batch is touched or any
  // kernel is launched: a refused call leaves the table as it found it
  for (Shard *m : members) {
    const int r = m->cfg.rank;
    HCTR_CHECK(grads[r] == nullptr || m->prev.n % bag == 0, "pooled push: the previous batch is not a whole number of bags");
    HCTR_CHECK(dsts[r] == nullptr || m->cur.n % bag == 0, "pooled pull: the batch is not a whole number of bags");
  }
  try {
    push_pull_steps(grads, dsts, bag);
  } catch (...) {
    // Something failed after work was enqueued (a runtime error, a device-side check).  Nothing may still be running
    // when the caller sees the error, and an index that this call started to join is handed back to the next call
    // that needs it (flush_index takes its results over) instead of being dropped with its batch.
    (void)hipStreamSynchronize(index_stream);
    (void)hipStreamSynchronize(stream);
    for (auto &mk : marks) {
      event_pool.push_back(mk.a);
      event_pool.push_back(mk.b);
    }
    marks.clear();
    if (index_joining_) index_pending = true;
    index_joining_ = false;
    throw;
  }
}

void Group::push_pull_steps(const float *const *grads, float *const *dsts, uint32_t bag) {
  if (time_calls) HCTR_HIP(hipEventRecord(ev0, stream));
  for (Shard *m : members) m->begin_push(grads[m->cfg.rank], bag);
  place_pushes();
  for (Shard *m : members)
    m->generate_gradient(nrank > 1 ? push_delta_dev.as<uint32_t>() + (size_t)nrank * m->cfg.rank : nullptr);
  if (time_calls) HCTR_HIP(hipEventRecord(ev_push, stream));
  if (nrank > 1) HCTR_HIP(hipEventRecord(ev_pushed, stream));
  enqueue_index_rest(); // the pushes are in their queue, now the rest of the current batches' index
  // One shard and a small batch: the gather works from the batch's keys and needs nothing of its index, which is
  // longer than the push of such a batch.  The step then leaves the index pending: whatever needs it next (the next
  // preprocess, which makes this batch the previous one; a fetch) waits for it, by then long done.
  const bool index_not_needed = nrank == 1 && (dsts[0] == nullptr || members[0]->direct_now(bag));
  const bool join_index = index_pending && !index_not_needed;
  uint64_t queries_max = 0;
  if (nrank > 1) {
    if (!owner_host) {
      HCTR_HIP(hipHostMalloc((void **)&owner_host, (size_t)nrank * sizeof(OwnerShard), hipHostMallocDefault));
      owner_dev.reserve((size_t)nrank * sizeof(OwnerShard));
      ret_delta_dev.reserve((size_t)nrank * nrank * sizeof(uint32_t));
    }
    queries_max = reserve_queries();
    for (Shard *m : members) m->fill_owner_args(owner_host[m->cfg.rank], queries_max);
    {
      // Behind the index, on its stream and beside the pushes: the owners' records go to the device and the receive
      // area of the queries is cut there from the counts the index left (nothing of this needs the host to know them).
      StreamSwitch on(*this, index_stream);
      HCTR_HIP(hipMemcpyAsync(owner_dev.p, owner_host, (size_t)nrank * sizeof(OwnerShard), hipMemcpyHostToDevice, stream));
      {
        StageScope st(*this, S_QUERY);
        launch_place_queries(stream, owner_dev.as<OwnerShard>(), owner_host, nrank, query_area());
      }
      HCTR_HIP(hipEventRecord(ev_index, stream));
      // the push plans of the current batches, for the step in which they are the previous ones: after the pushes of
      // this step (they move the update counters the plan reads), beside everything else the step still does
      HCTR_HIP(hipStreamWaitEvent(stream, ev_pushed, 0));
      for (Shard *m : members) m->plan_batch(m->cur);
      HCTR_HIP(hipEventRecord(ev_plan, stream));
    }
  }
  if (join_index) {
    // The push kernels are in the main stream's queue; everything below needs the index of the current batches, still
    // running or done on the second stream.  The host does not wait for it (the reference has the shapes on the host
    // because its preprocess waits for all of its work, csrc/core/hetu_gpu_table.cu:60-64): what the index leaves --
    // unique keys per shard, queries per owner -- is read on the device by the kernels that need it, and by the host
    // when the step is over.
    index_pending = false;
    index_joining_ = true;
  }
  if (join_index || nrank > 1) HCTR_HIP(hipStreamWaitEvent(stream, ev_index, 0));
  if (nrank > 1) {
    for (Shard *m : members) m->generate_query(query_delta_dev.as<uint32_t>() + (size_t)nrank * m->cfg.rank);
    owner_side(queries_max);
    // the reference waits here for the return counts (hetu_gpu_table.cu:33); they stay on the device
  }
  for (Shard *m : members) m->write_back(dsts[m->cfg.rank], bag);
  if (time_calls) HCTR_HIP(hipEventRecord(ev1, stream));
  if (nrank > 1) HCTR_HIP(hipStreamWaitEvent(stream, ev_plan, 0));
  sync_stream();
  collect_marks();
  if (nrank > 1)
    for (Shard *m : members) m->finish_plan(m->cur);
  if (join_index) {
    index_joining_ = false; // from here on the results are taken over, or the batch's own error is reported
    if (nrank == 1) members[0]->finish_preprocess();
    else
      for (Shard *m : members) m->finish_index();
    exchange_shapes();
  }
  if (nrank > 1) note_query_places();
  float ms = 0.f, push_ms = 0.f;
  if (time_calls) {
    HCTR_HIP(hipEventElapsedTime(&ms, ev0, ev1));
    HCTR_HIP(hipEventElapsedTime(&push_ms, ev0, ev_push));
  }
  std::string first_error;
  for (Shard *m : members) {
    m->last_pp_ms = ms;
    m->last_push_ms = push_ms;
    try {
      if (nrank > 1) m->finish_handle_query();
      m->finish_push_pull();
    } catch (const Error &e) {
      if (first_error.empty()) first_error = e.what();
    }
  }
  if (!first_error.empty()) throw Error(first_error);
}

// Rendezvous of the nrank per-shard callers: the last one to arrive runs the step for all.
template <typename F> void Group::collective(int rank, int op, F &&run_all) {
  std::unique_lock<std::mutex> lk(mu_);
  if (arrived_ > 0 && pending_op_ != op)
    throw Error("hetuCTR: shards of one group are in different calls (preprocess vs push_pull)");
  pending_op_ = op;
  arrived_++;
  if (arrived_ == nrank) {
    failure_.clear();
    try {
      run_all();
    } catch (const std::exception &e) {
      failure_ = e.what();
    }
    arrived_ = 0;
    generation_++;
    cv_.notify_all();
  } else {
    const uint64_t gen = generation_;
    const bool ok = cv_.wait_for(lk, std::chrono::duration<double>(wait_seconds), [&] { return generation_ != gen; });
    if (!ok) {
      arrived_--;
      throw Error("hetuCTR: timed out waiting for the other shards of the group to make the same call");
    }
  }
  if (!failure_.empty()) throw Error(failure_);
}

void Group::preprocess_one(int rank, const int64_t *keys, size_t n) {
  if (nrank == 1) {
    preprocess_all(&keys, &n);
    return;
  }
  {
    std::lock_guard<std::mutex> lk(mu_);
    a_keys_[rank] = keys;
    a_n_[rank] = n;
  }
  collective(rank, 1, [&] { preprocess_all(a_keys_.data(), a_n_.data()); });
}

void Group::push_pull_one(int rank, const float *grad, float *dst, size_t bag) {
  if (nrank == 1) {
    push_pull_all(&grad, &dst, bag);
    return;
  }
  {
    std::lock_guard<std::mutex> lk(mu_);
    a_grad_[rank] = grad;
    a_dst_[rank] = dst;
    a_bag_[rank] = bag;
  }
  collective(rank, 2, [&] {
    for (int r = 1; r < nrank; r++)
      HCTR_CHECK(a_bag_[r] == a_bag_[0], "the shards of a group must pool with the same bag size");
    push_pull_all(a_grad_.data(), a_dst_.data(), a_bag_[0]);
  });
}

// ---- registry of groups by (ip, port) --------------------------------------------------------------
static std::mutex g_registry_mu;
static std::map<std::string, std::weak_ptr<Group>> g_registry;

std::shared_ptr<Group> find_or_create_group(int nrank, int device_id, const std::string &ip, int port) {
  if (nrank == 1) return std::make_shared<Group>(1, device_id, "");
  const std::string key = ip + ":" + std::to_string(port);
  std::lock_guard<std::mutex> lk(g_registry_mu);
  auto it = g_registry.find(key);
  if (it != g_registry.end()) {
    if (auto g = it->second.lock()) {
      HCTR_CHECK(g->nrank == nrank, "a group with this (ip, port) exists with a different nrank");
      HCTR_CHECK(g->device_id == device_id, "all shards of a loopback group live on one device");
      return g;
    }
  }
  auto g = std::make_shared<Group>(nrank, device_id, key);
  g_registry[key] = g;
  return g;
}

} // namespace hctr
