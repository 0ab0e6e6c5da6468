/*
 * C ABI of the MI355X (gfx950) implementation of HetuCTR's per-GPU embedding hot path.
 *
 * This is the boundary a binding of the reference's table API sits on: plain pointers and sizes,
 * an opaque handle, an int status (0 = ok) and a per-thread error string.  No torch, pybind or C++
 * types cross it.  The python module `hetuCTR` (same surface as the reference's
 * csrc/pybind/pybind.cu:42-79) is a thin pybind11 layer over exactly these entry points.
 *
 * Citations are relative to the reference tree.
 */
#ifndef HETUCTR_HIP_H_
#define HETUCTR_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hctr_table hctr_table;

/* hetuCTR::InitType, csrc/utils/initializer.h:8-14 (same numeric order) */
enum { HCTR_INIT_ZERO = 0, HCTR_INIT_NORMAL = 1, HCTR_INIT_UNIFORM = 2, HCTR_INIT_TRUNCATED_NORMAL = 3 };

/* Constructor arguments of hetuCTR::HetuTable, csrc/core/hetu_gpu_table.h:109-124 /
 * csrc/pybind/pybind.cu:63-69, in the same order. */
typedef struct hctr_config {
  int rank;            /* this shard's rank, 0 <= rank < nrank */
  int nrank;           /* number of shards, <= 256 (worker ids are one byte, csrc/core/types.h:28) */
  int device_id;       /* HIP device ordinal */
  const char *ip;      /* with nrank > 1: (ip, port) names the in-process loopback group the table joins */
  int port;            /*   (the reference uses them for its NCCL rendezvous, table_initialize.cu:14-31) */
  size_t length;       /* kEmbeddingIDMax: ids are 0 .. length-1 */
  size_t width;        /* kEmbeddingWidth: floats per row */
  long long pull_bound;
  long long push_bound;
  int init_type;       /* HCTR_INIT_* */
  float init_a;        /* mean, or lower bound */
  float init_b;        /* stddev, or upper bound */
  float learning_rate;
  int verbose;
} hctr_config;

/* Replaces HetuTable::HetuTable + initializeTable + initialize
 * (csrc/core/table_initialize.cu:66-164, csrc/utils/initializer.cu:94-103).
 * root_arr: `length` owner bytes; storage_arr: the ids resident on this shard (owned and cached),
 * both HOST pointers read only during the call.  Every id owned by `rank` must be in storage_arr. */
int hctr_create(const hctr_config *cfg, const uint8_t *root_arr, const int64_t *storage_arr, size_t n_storage,
                hctr_table **out);

/* Replaces HetuTable::~HetuTable (csrc/core/table_initialize.cu:231-245). */
int hctr_destroy(hctr_table *t);

/* Replaces HetuTable::preprocess (csrc/core/hetu_gpu_table.cu:43-65): the previous batch becomes the
 * one whose gradients come next, `keys` (int64[n], HOST OR DEVICE memory) becomes the current batch.
 * The call returns when the caller's ids have been read (the buffer may be reused at once) and any error in them has
 * been reported; sorting and deduplicating them goes on behind the return and is waited for by whatever needs it
 * next (hctr_push_pull, a second hctr_preprocess, hctr_debug_fetch).  This is the one deviation from the reference,
 * whose call returns when all of its work is done (hetu_gpu_table.cu:64): hctr_defer_index(t, 0), or
 * HETUCTR_DEFER_INDEX=0 in the environment, restores exactly that.  The details of the early return are with
 * hctr_defer_index below.  With nrank > 1 the call completes when every shard of the group has made it. */
int hctr_preprocess(hctr_table *t, const int64_t *keys, size_t n);

/* hctr_preprocess for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same result as hctr_preprocess with the early return switched off:
 * like the reference's call it returns when all its work is done.  It calls no hipMalloc / hipFree and no allocating
 * routine; it does synchronise the table's stream and reads counts back to the host, so it cannot be recorded into a
 * HIP graph:
 *   - the index scratch (sort ping-pong buffers, per-tile digit tables, scan sums, head counts) lives in a static device array of
 *     7.1 MiB that every GPU the library runs on holds until the process ends;
 *   - n is at most 262144 keys (HCTR_NOALLOC_MAX_KEYS), larger batches are refused;
 *   - keys must be DEVICE memory (ids in pageable host memory go through a pinned staging buffer the library
 *     would have to allocate);
 *   - the table has one shard, and its two batch buffers already hold n keys: they are sized by ordinary
 *     hctr_preprocess calls (two in a row with the largest batch size both); otherwise the call is refused.
 * All tables on one GPU share that GPU's array: calls that overlap on one GPU race. */
#define HCTR_NOALLOC_MAX_KEYS 262144
int hctr_preprocess_noalloc(hctr_table *t, const int64_t *keys, size_t n);

/* Replaces HetuTable::pushPull (csrc/core/hetu_gpu_table.cu:9-41).  grad: DEVICE float[n_prev][width]
 * for the batch before the current one, or NULL (inference: nothing is pushed).  dst: DEVICE
 * float[n][width] receives the rows of the current batch.  Synchronous. */
int hctr_push_pull(hctr_table *t, const float *grad, float *dst);

/* hctr_push_pull for multi-hot lookups that are sum-pooled: the batch is a sequence of bags of `bag` consecutive keys
 * (the layout the reference's drivers give a multi-hot field, tests/benchmark.py:19-23 flattens samples the same
 * way).  No counterpart in the reference, whose API has no pooling: there a bag is just more keys, the caller adds the
 * pulled rows up itself and hands back the bag's gradient once per key.  Here dst_pooled is DEVICE
 * float[n / bag][width], row b = the rows of keys b*bag .. b*bag+bag-1 added in that order (fp32, starting from the
 * first), and grad_pooled is DEVICE float[n_prev / bag][width] or NULL, every key of a bag receiving its bag's row;
 * the table ends in exactly the state hctr_push_pull reaches with the replicated gradients.  bag = 1 is
 * hctr_push_pull; n and n_prev must be multiples of bag.  The pooled forms move 1/bag of the gradient and output
 * bytes. */
int hctr_push_pull_pooled(hctr_table *t, const float *grad_pooled, float *dst_pooled, size_t bag);

/* Single-caller forms of the two calls above for a whole loopback group: entry r of each array belongs
 * to tables[r], which must be rank r of one complete group.  What R reference processes do in
 * lock-step with NCCL between the stages (csrc/core/all2all.cu:6-130) happens inside one call. */
int hctr_group_preprocess(hctr_table *const *tables, int nrank, const int64_t *const *keys, const size_t *n);
int hctr_group_push_pull(hctr_table *const *tables, int nrank, const float *const *grads, float *const *dsts);
int hctr_group_push_pull_pooled(hctr_table *const *tables, int nrank, const float *const *grads_pooled,
                                float *const *dsts_pooled, size_t bag);

/* Replaces the module function hetuCTR.seed (csrc/pybind/pybind.cu:77): seed of tables created later. */
void hctr_seed(unsigned long seed);

/* Replace HetuTable::debugString / debugStringFull (csrc/core/debug.cu:5-24).  Return the length
 * the full string needs (excluding the terminator); write at most cap bytes including it. */
int hctr_repr(hctr_table *t, char *buf, size_t cap);
int hctr_debug(hctr_table *t, char *buf, size_t cap);

/* Message of the last failed call on this thread (the reference prints and exits instead,
 * csrc/common/helper_cuda.h:586-599). */
const char *hctr_last_error(void);

/* Introspection of the integer intermediates and of the table state; the reference exposes none
 * (csrc/pybind/pybind.cu:62-75) although they are what its kernels compute
 * (csrc/core/preprocess_struct.h:7-24, csrc/core/hetu_gpu_table.h:38-70).  `which` is HCTR_F_*;
 * *n_elems receives the element count; at most cap_elems elements are written to host_out.
 * Integer items are int64, HCTR_F_EMBEDDING and HCTR_F_PENDING are float. */
enum {
  HCTR_F_UNIQUE = 0, HCTR_F_SORTED_ARG = 1, HCTR_F_RUN_START = 2, HCTR_F_IDX_MAP = 3, HCTR_F_ROOT = 4,
  HCTR_F_OFFSET = 5, HCTR_F_SEND_CNT = 6, HCTR_F_RECV_CNT = 7, HCTR_F_NEED_UPDATE = 8, HCTR_F_UPDATE_PREFIX = 9,
  HCTR_F_PUSH_CNT = 10, HCTR_F_PUSHRECV_CNT = 11, HCTR_F_OUTDATED = 12, HCTR_F_GOT = 13, HCTR_F_VERSION = 14,
  HCTR_F_UPDATES = 15, HCTR_F_EMBEDDING = 16, HCTR_F_PENDING = 17, HCTR_F_STORE_IDS = 18, HCTR_F_STATS = 19,
  HCTR_F_SIZES = 20, HCTR_F_KEYS = 21
};
int hctr_debug_fetch(hctr_table *t, int which, void *host_out, size_t cap_elems, size_t *n_elems);

/* Checkpoint of one shard.  No counterpart in the reference, whose table state lives in device memory only
 * (csrc/core/hetu_gpu_table.h:38-70, freed in csrc/core/table_initialize.cu:231-245).  hctr_save writes the resident
 * rows, their versions and, for cached rows, the pending gradients and update counters to `path` (one file per
 * shard; format in hetuctr_amd/csrc/checkpoint.hip).  hctr_load restores them into a table created with the same
 * rank, nrank, length, width, root_arr and storage_arr (checked; bounds and learning rate are the new table's) and
 * empties its two batches: the next hctr_push_pull pushes nothing, as after hctr_create.  Call both between steps,
 * from every shard of a group. */
int hctr_save(hctr_table *t, const char *path);
int hctr_load(hctr_table *t, const char *path);

/* The HIP stream (hipStream_t) every kernel of this table's group is launched on, for callers that time
 * or order work against it (the reference's stream_main_, csrc/core/hetu_gpu_table.h:40). */
int hctr_stream(hctr_table *t, void **stream_out);

/* Device time of the last preprocess and push_pull calls in milliseconds, measured with HIP events on
 * that stream around the launched work (host-side waits excluded).  The events cost host time in every call, so they
 * are recorded only while hctr_call_timing(t, 1) is in force (off when a table is created; switching it either way
 * zeroes the stored times).  While it is off hctr_last_times and hctr_last_push_ms fail with an error instead of
 * returning stale or zero times.  No counterpart in the reference. */
int hctr_call_timing(hctr_table *t, int on);
int hctr_last_times(hctr_table *t, float *preprocess_ms, float *push_pull_ms);

/* hctr_preprocess returns as soon as the caller's ids have been read (the buffer may be reused).  With several shards
 * the push plan of the previous batch was made at the end of the step before (only a batch that no hctr_push_pull has
 * seen, e.g. after two hctr_preprocess calls in a row, is planned, and waited for, in this call).  The sort / unique
 * stages of the new batch keep running on a
 * second stream, next to the gradient push that the following hctr_push_pull starts, and are waited for before the
 * rows are gathered (several shards: before the queries are built).  preprocess_ms above is then the time up to
 * that return, push_pull_ms covers the rest.  Anything that needs the batch's index earlier (a second hctr_preprocess,
 * hctr_debug_fetch, hctr_stage_timing) waits for it.  HETUCTR_DEFER_INDEX=0 in the environment restores a
 * preprocess that returns only when all its work is done (hetu_gpu_table.cu:64); with stage timing on it always is.
 * hctr_last_push_ms (needs hctr_call_timing, like hctr_last_times): device time from the start of the last hctr_push_pull to the end of its push stage, i.e. the
 * push kernel while the index of the next batch runs beside it.  No counterpart in the reference. */
int hctr_last_push_ms(hctr_table *t, float *push_ms);
/* The same switch as HETUCTR_DEFER_INDEX for a table's group at run time: 0 makes hctr_preprocess return only when
 * all of its work is done (the reference's contract, hetu_gpu_table.cu:64), non-zero restores the early return. */
int hctr_defer_index(hctr_table *t, int on);

/* Per-stage device time.  hctr_stage_timing(t, 1) resets the accumulators and makes every later call bracket
 * each stage's launches with HIP events on the table's stream; hctr_stage_times returns, per stage, the
 * accumulated milliseconds and the number of bracketed intervals.  Stage i is named hctr_stage_name(i),
 * 0 <= i < hctr_stage_count().  No counterpart in the reference, which is profiled from outside with nvprof
 * (tests/run.sh:4). */
int hctr_stage_timing(hctr_table *t, int on);
int hctr_stage_count(void);
const char *hctr_stage_name(int stage);
int hctr_stage_times(hctr_table *t, double *ms_total, long long *launches, int cap);

/* Measurement aid without a counterpart in the reference: copies `bytes` (a multiple of 16) of device memory with a
 * plain 16-byte-lane kernel on the default stream, 1 + repeats times, and reports the average duration.  A launch
 * reads and writes exactly `bytes`, which is what hardware byte counters are scaled against. */
int hctr_copy_probe(void *dst, const void *src, size_t bytes, int repeats, float *ms_avg);

/* Batch sampling from a click log in device memory: keys_out[r * n_fields + f] = log[rows[r] * n_fields + f], i.e.
 * data[idx].flatten() of the reference's benchmark driver (tests/benchmark.py:19-23) for an int64 log of
 * n_samples x n_fields ids (the array its Criteo loader returns, tests/benchmark.py:26-31).  All three pointers are
 * DEVICE memory; runs on the default stream and returns when the ids are written, ready for hctr_preprocess. */
int hctr_sample_rows(const int64_t *log, size_t n_samples, size_t n_fields, const int64_t *rows, size_t n_rows,
                     int64_t *keys_out);

/* ---- offline partitioner ---------------------------------------------------------------------------------------
 * The C surface under the python module hetuCTR_partition (csrc/partition/pybind.cc:6-25).  Results are those of the
 * reference's PartitionStruct run without OpenMP threads: samples and embeddings visited in index order, every move
 * applied before the next decision (with threads the reference's sweeps race on their shared counters and its result
 * is not a function of its input).  All pointers are HOST pointers. */
typedef struct hctr_partition hctr_partition;

/* Replaces partition() / PartitionStruct::PartitionStruct (csrc/partition/partition.cc:26-87,196-206).
 * data: n_data x n_slot embedding ids, row-major; comm_mat: n_part x n_part, comm_mat[i][j] = cost for part i of
 * fetching a row owned by part j.  The initial assignment is the one the reference draws from the C library's
 * rand(); seed is what srand() would have been given (the reference never seeds: 1). */
int hctr_part_create(const int32_t *data, size_t n_data, size_t n_slot, const float *comm_mat, int n_part,
                     int batch_size, unsigned seed, hctr_partition **out);
int hctr_part_destroy(hctr_partition *h);
/* n_embed = largest id + 1 (partition.cc:33-37) */
int hctr_part_sizes(hctr_partition *h, size_t *n_data, size_t *n_embed, int *n_part);
/* PartitionStruct::refineData / refineEmbed (partition.cc:89-120 / 122-166): one sweep over the samples / embeddings */
int hctr_part_refine_data(hctr_partition *h);
int hctr_part_refine_embed(hctr_partition *h);
/* PartitionStruct::getCommunication (partition.cc:168-181): cost[n_part * n_part] */
int hctr_part_get_communication(hctr_partition *h, float *cost);
/* PartitionStruct::getPriority (partition.cc:183-194): priority[n_part * n_embed] */
int hctr_part_get_priority(hctr_partition *h, float *priority);
/* get_result / get_data_cnt / get_embed_cnt (pybind.cc:13-21); any pointer may be NULL */
int hctr_part_get_result(hctr_partition *h, int32_t *data_part, int32_t *embed_part);
int hctr_part_get_counts(hctr_partition *h, int32_t *data_cnt, int32_t *embed_cnt);
/* The cache candidates the reference's driver script derives from the priorities with one numpy argsort per part
 * (experimental/partition.py:51-57): per part, the embeddings it does not own by descending priority; equal
 * priorities, whose order numpy leaves open, by descending id.  Runs on the current HIP device (priorities, one radix
 * sort per part).  lists[part * max_len + q], lens[part] <= max_len entries each; kernel_ms (may be NULL) receives
 * the device time between the first and the last kernel. */
int hctr_part_cache_lists(hctr_partition *h, size_t max_len, int32_t *lists, size_t *lens, float *kernel_ms);

/* Version string of the library. */
const char *hctr_version(void);

#ifdef __cplusplus
}
#endif
#endif /* HETUCTR_HIP_H_ */
