// extern "C" surface declared in include/hetuctr_hip.h.  Exceptions never cross it: every entry point returns
// 0 or stores a message for hctr_last_error() and returns 1.
#include <atomic>
#include <cstdio>
#include <cstring>

#include "partition.h"
#include "table.h"

using namespace hctr;

struct hctr_table {
  Shard *shard;
};

struct hctr_partition {
  Partitioner *p;
};

namespace {
thread_local std::string g_error;
std::atomic<unsigned long> g_seed{0}; // hetuCTR::__seed, csrc/core/hetu_gpu_table.cu:7

template <typename F> int guarded(F &&f) {
  try {
    f();
    return 0;
  } catch (const std::exception &e) {
    g_error = e.what();
  } catch (...) {
    g_error = "hetuCTR: unknown error";
  }
  return 1;
}

int write_string(const std::string &s, char *buf, size_t cap) {
  if (buf && cap) {
    const size_t n = std::min(cap - 1, s.size());
    memcpy(buf, s.data(), n);
    buf[n] = 0;
  }
  return (int)s.size();
}
} // namespace

extern "C" {
#pragma GCC visibility push(default)

const char *hctr_last_error(void) { return g_error.c_str(); }
const char *hctr_version(void) { return "hetuctr-hip 0.1 (gfx950)"; }
void hctr_seed(unsigned long seed) { g_seed = seed; }

int hctr_create(const hctr_config *cfg, const uint8_t *root_arr, const int64_t *storage_arr, size_t n_storage,
                hctr_table **out) {
  return guarded([&] {
    HCTR_CHECK(cfg && out, "null argument");
    *out = nullptr;
    HCTR_CHECK(cfg->nrank >= 1 && cfg->nrank <= 256, "nrank must be in 1..256 (worker ids are one byte)");
    auto group = find_or_create_group(cfg->nrank, cfg->device_id, cfg->ip ? cfg->ip : "", cfg->port);
    // the reference passes the global seed as an unsigned int (table_initialize.cu:156, initializer.h:37)
    Shard *s = new Shard(*cfg, root_arr, storage_arr, n_storage, (unsigned)g_seed.load(), group);
    try {
      group->join(s);
    } catch (...) {
      delete s;
      throw;
    }
    if (cfg->verbose >= 1)
      printf("HetuTable rank %d: Table Init Successfully (%zu rows resident, %u cached)\n", cfg->rank, n_storage,
             s->tv.n_cached);
    *out = new hctr_table{s};
  });
}

int hctr_destroy(hctr_table *t) {
  return guarded([&] {
    if (!t) return;
    if (t->shard) {
      (void)hipSetDevice(t->shard->cfg.device_id);
      (void)hipStreamSynchronize(t->shard->group->stream);
      t->shard->group->leave(t->shard);
      delete t->shard;
    }
    delete t;
  });
}

int hctr_preprocess(hctr_table *t, const int64_t *keys, size_t n) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->group->preprocess_one(t->shard->cfg.rank, keys, n);
  });
}

int hctr_preprocess_noalloc(hctr_table *t, const int64_t *keys, size_t n) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->group->preprocess_noalloc(keys, n);
  });
}

int hctr_push_pull(hctr_table *t, const float *grad, float *dst) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->group->push_pull_one(t->shard->cfg.rank, grad, dst);
  });
}

int hctr_push_pull_pooled(hctr_table *t, const float *grad_pooled, float *dst_pooled, size_t bag) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->group->push_pull_one(t->shard->cfg.rank, grad_pooled, dst_pooled, bag);
  });
}

static Group *group_of(hctr_table *const *tables, int nrank) {
  HCTR_CHECK(tables && nrank >= 1, "null table list");
  for (int r = 0; r < nrank; r++) HCTR_CHECK(tables[r] && tables[r]->shard, "null table");
  Group *g = tables[0]->shard->group.get();
  HCTR_CHECK(g->nrank == nrank, "the table list must hold every rank of the group");
  for (int r = 0; r < nrank; r++)
    HCTR_CHECK(tables[r]->shard->group.get() == g && tables[r]->shard->cfg.rank == r,
               "tables[r] must be rank r of one group");
  return g;
}

int hctr_group_preprocess(hctr_table *const *tables, int nrank, const int64_t *const *keys, const size_t *n) {
  return guarded([&] { group_of(tables, nrank)->preprocess_all(keys, n); });
}

int hctr_group_push_pull(hctr_table *const *tables, int nrank, const float *const *grads, float *const *dsts) {
  return guarded([&] { group_of(tables, nrank)->push_pull_all(grads, dsts); });
}

int hctr_group_push_pull_pooled(hctr_table *const *tables, int nrank, const float *const *grads_pooled,
                                float *const *dsts_pooled, size_t bag) {
  return guarded([&] { group_of(tables, nrank)->push_pull_all(grads_pooled, dsts_pooled, bag); });
}

// csrc/core/debug.cu:5-12
int hctr_repr(hctr_table *t, char *buf, size_t cap) {
  if (!t || !t->shard) return -1;
  char b[256];
  const Shard &s = *t->shard;
  snprintf(b, sizeof b, "<HetuTable root/store/all=%ld/%ld/%ld>", (long)(s.tv.n_stored - s.tv.n_cached),
           (long)s.tv.n_stored, (long)s.tv.id_max);
  return write_string(b, buf, cap);
}

// csrc/core/debug.cu:14-24
int hctr_debug(hctr_table *t, char *buf, size_t cap) {
  if (!t || !t->shard) return -1;
  char b[512];
  const Shard &s = *t->shard;
  snprintf(b, sizeof b, "<HetuTable root/store/all=%ld/%ld/%ld rank=%d nrank=%d device_id=%d width=%ld push/pull=%lld/%lld>",
           (long)(s.tv.n_stored - s.tv.n_cached), (long)s.tv.n_stored, (long)s.tv.id_max, s.cfg.rank, s.cfg.nrank,
           s.cfg.device_id, (long)s.tv.width, (long long)s.tv.push_bound, (long long)s.tv.pull_bound);
  return write_string(b, buf, cap);
}

int hctr_debug_fetch(hctr_table *t, int which, void *host_out, size_t cap_elems, size_t *n_elems) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    const size_t n = t->shard->fetch(which, host_out, host_out ? cap_elems : 0);
    if (n_elems) *n_elems = n;
  });
}

int hctr_save(hctr_table *t, const char *path) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->save(path);
  });
}

int hctr_load(hctr_table *t, const char *path) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->load(path);
  });
}

int hctr_stream(hctr_table *t, void **stream_out) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard && stream_out, "null argument");
    *stream_out = (void *)t->shard->group->stream;
  });
}

int hctr_call_timing(hctr_table *t, int on) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->group->set_call_timing(on != 0);
  });
}

int hctr_last_times(hctr_table *t, float *preprocess_ms, float *push_pull_ms) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    HCTR_CHECK(t->shard->group->time_calls, "call timing is off: switch it on with hctr_call_timing(t, 1) first");
    if (preprocess_ms) *preprocess_ms = t->shard->last_pre_ms;
    if (push_pull_ms) *push_pull_ms = t->shard->last_pp_ms;
  });
}

int hctr_last_push_ms(hctr_table *t, float *push_ms) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard && push_ms, "null argument");
    HCTR_CHECK(t->shard->group->time_calls, "call timing is off: switch it on with hctr_call_timing(t, 1) first");
    *push_ms = t->shard->last_push_ms;
  });
}

int hctr_stage_timing(hctr_table *t, int on) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->group->set_stage_timing(on != 0);
  });
}

int hctr_defer_index(hctr_table *t, int on) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    t->shard->group->set_defer_index(on != 0);
  });
}

int hctr_stage_count(void) { return S_COUNT; }
const char *hctr_stage_name(int stage) { return stage_name(stage); }

int hctr_stage_times(hctr_table *t, double *ms_total, long long *launches, int cap) {
  return guarded([&] {
    HCTR_CHECK(t && t->shard, "null table");
    Group &g = *t->shard->group;
    for (int i = 0; i < S_COUNT && i < cap; i++) {
      if (ms_total) ms_total[i] = g.stage_ms[i];
      if (launches) launches[i] = g.stage_calls[i];
    }
  });
}

int hctr_copy_probe(void *dst, const void *src, size_t bytes, int repeats, float *ms_avg) {
  return guarded([&] {
    HCTR_CHECK(dst && src && bytes % 16 == 0 && repeats >= 1, "copy probe: device pointers, bytes a multiple of 16");
    hipEvent_t a, b;
    HCTR_HIP(hipEventCreate(&a));
    HCTR_HIP(hipEventCreate(&b));
    launch_plain_copy(nullptr, src, dst, bytes); // untimed first launch
    HCTR_HIP(hipEventRecord(a, nullptr));
    for (int i = 0; i < repeats; i++) launch_plain_copy(nullptr, src, dst, bytes);
    HCTR_HIP(hipEventRecord(b, nullptr));
    HCTR_HIP(hipEventSynchronize(b));
    float ms = 0.f;
    HCTR_HIP(hipEventElapsedTime(&ms, a, b));
    if (ms_avg) *ms_avg = ms / repeats;
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
  });
}

int hctr_sample_rows(const int64_t *log, size_t n_samples, size_t n_fields, const int64_t *rows, size_t n_rows,
                     int64_t *keys_out) {
  return guarded([&] {
    HCTR_CHECK(n_rows == 0 || (log && rows && keys_out), "null argument");
    HCTR_CHECK(n_fields >= 1 && n_fields < (1u << 20), "fields out of range");
    if (!n_rows) return;
    uint32_t *err = nullptr;
    HCTR_HIP(hipMalloc((void **)&err, 4));
    uint32_t h = 0;
    hipError_t e = hipMemsetAsync(err, 0, 4, nullptr);
    try {
      HCTR_HIP(e);
      launch_sample_rows(nullptr, (const index_t *)log, n_samples, (uint32_t)n_fields, (const index_t *)rows, n_rows,
                         (index_t *)keys_out, err);
      HCTR_HIP(hipMemcpy(&h, err, 4, hipMemcpyDeviceToHost)); // waits for the kernel
    } catch (...) {
      (void)hipFree(err);
      throw;
    }
    (void)hipFree(err);
    HCTR_CHECK(h == 0, "sample_rows: a row number lies outside [0, n_samples) (its ids were written as 0)");
  });
}

int hctr_part_create(const int32_t *data, size_t n_data, size_t n_slot, const float *comm_mat, int n_part,
                     int batch_size, unsigned seed, hctr_partition **out) {
  return guarded([&] {
    HCTR_CHECK(out, "null argument");
    *out = nullptr;
    *out = new hctr_partition{new Partitioner(data, n_data, n_slot, comm_mat, n_part, batch_size, seed)};
  });
}

int hctr_part_destroy(hctr_partition *h) {
  return guarded([&] {
    if (!h) return;
    delete h->p;
    delete h;
  });
}

int hctr_part_sizes(hctr_partition *h, size_t *n_data, size_t *n_embed, int *n_part) {
  return guarded([&] {
    HCTR_CHECK(h && h->p, "null partition");
    if (n_data) *n_data = h->p->n_data;
    if (n_embed) *n_embed = h->p->n_embed;
    if (n_part) *n_part = h->p->n_part;
  });
}

int hctr_part_refine_data(hctr_partition *h) {
  return guarded([&] {
    HCTR_CHECK(h && h->p, "null partition");
    h->p->refine_data();
  });
}

int hctr_part_refine_embed(hctr_partition *h) {
  return guarded([&] {
    HCTR_CHECK(h && h->p, "null partition");
    h->p->refine_embed();
  });
}

int hctr_part_get_communication(hctr_partition *h, float *cost) {
  return guarded([&] {
    HCTR_CHECK(h && h->p && cost, "null argument");
    h->p->communication(cost);
  });
}

int hctr_part_get_priority(hctr_partition *h, float *priority) {
  return guarded([&] {
    HCTR_CHECK(h && h->p && priority, "null argument");
    h->p->priority(priority);
  });
}

int hctr_part_get_result(hctr_partition *h, int32_t *data_part, int32_t *embed_part) {
  return guarded([&] {
    HCTR_CHECK(h && h->p, "null partition");
    if (data_part) memcpy(data_part, h->p->res_data.data(), h->p->n_data * sizeof(int32_t));
    if (embed_part) memcpy(embed_part, h->p->res_embed.data(), h->p->n_embed * sizeof(int32_t));
  });
}

int hctr_part_get_counts(hctr_partition *h, int32_t *data_cnt, int32_t *embed_cnt) {
  return guarded([&] {
    HCTR_CHECK(h && h->p, "null partition");
    if (data_cnt) memcpy(data_cnt, h->p->cnt_data.data(), h->p->n_part * sizeof(int32_t));
    if (embed_cnt) memcpy(embed_cnt, h->p->cnt_embed.data(), h->p->n_part * sizeof(int32_t));
  });
}

int hctr_part_cache_lists(hctr_partition *h, size_t max_len, int32_t *lists, size_t *lens, float *kernel_ms) {
  return guarded([&] {
    HCTR_CHECK(h && h->p, "null partition");
    h->p->cache_lists(max_len, lists, lens, kernel_ms);
  });
}

#pragma GCC visibility pop
} // extern "C"
