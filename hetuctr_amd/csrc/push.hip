// Gradient push: deterministic segment-sum of the gradient rows of every unique key of the previous
// batch, fused with the SGD write-back to the table, the hot-row cache, the pending-gradient store,
// the version / update counters and the push buffer.
// Reference: csrc/core/generate_query.cu:8-89 (gradient_reduction_kernel, gradient_index_kernel).
//
// Summation order: the reference adds the gradient rows of one key serially, in ascending batch position,
// then multiplies once by -lr and adds once to the row.  fp32 addition is not associative, so any other
// order differs from it in the last bits by an amount that grows with the number of duplicates.  Here
// every run of equal keys is summed by ONE chain of additions per column, in exactly that order: sums are
// bit-identical to the reference's order (compiled without fused multiply-add contraction), for any skew.
// "Bit-identical" is against that non-contracted restatement on the CPU: the reference itself is built by nvcc,
// whose default may fuse `sum *= -lr; dest += sum` (generate_query.cu:37-39) into one multiply-add, so against a
// CUDA build the last rounding of an updated value can differ by one ulp.  The contract against the reference is
// its own tolerance, 1e-5 relative.
//
// One launch, three ranges of blocks, one per class of run length (the long chains are dispatched first and the
// other blocks fill the machine behind them):
//  * long (> kLongRun duplicates): bundles of runs are streamed by whole blocks, one column slice at a time.  Seven
//    loader waves keep several 16-byte loads of gradient rows in flight each and stage them through a ring of
//    LDS slots; the first wave adds the staged rows in order, one column per lane.  The serial chain costs a
//    quarter of an LDS read and one add per duplicate while the memory latency is covered by the whole block.
//    The longest runs are started first and cut into narrower slices, i.e. fed by more blocks.
//  * medium (kTinyRun < duplicates <= kLongRun): one group of LPR lanes per run, kBatch rows in flight.
//  * short (<= kTinyRun): a group of LPR lanes (LPR*VEC floats = one row) owns a few consecutive unique keys
//    and sums their runs, all first loads of the group issued together.
#include <algorithm>
#include "kernels.h"

namespace hctr {

// tuning knobs (overridable at compile time for experiments)
#ifndef HCTR_TILE_BATCH
#define HCTR_TILE_BATCH 8
#endif
#ifndef HCTR_DEPTH
#define HCTR_DEPTH 8
#endif
#ifndef HCTR_RPT
#define HCTR_RPT 2
#endif
#ifndef HCTR_SLICE
#define HCTR_SLICE 64
#endif
#ifndef HCTR_LONG_BLOCKS
#define HCTR_LONG_BLOCKS 128
#endif
#ifndef HCTR_MED_BLOCKS
#define HCTR_MED_BLOCKS 512
#endif
constexpr int kPushBlock = 512;

constexpr int kBatch = HCTR_TILE_BATCH;   // short role: gradient rows in flight per group past the first two
constexpr int kDepth = HCTR_DEPTH;        // long role: chunks in flight per loader thread
constexpr int kRPT = HCTR_RPT;            // long role: rows per loader thread and chunk
#ifndef HCTR_SLOTS
#define HCTR_SLOTS 3
#endif
constexpr int kSlots = HCTR_SLOTS;        // long role: LDS ring slots
constexpr int kSlice = HCTR_SLICE;        // long role: columns per block
constexpr int kLongBlocks = HCTR_LONG_BLOCKS;
#ifndef HCTR_GIANT_SLICE
#define HCTR_GIANT_SLICE 32
#endif
#ifndef HCTR_GIANT_CLASSES
#define HCTR_GIANT_CLASSES 6
#endif
constexpr int kGiantSlice = HCTR_GIANT_SLICE;     // long role: the longest runs are cut into slices of this many columns;
constexpr int kGiantClasses = HCTR_GIANT_CLASSES; // they are the runs of the first length classes (>= 4096)
static_assert(kSlice % kGiantSlice == 0, "tiers of the long role");
constexpr int kMedBlocks = HCTR_MED_BLOCKS;

namespace {

__device__ __forceinline__ uint32_t div_up_dev(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

#ifndef HCTR_GRAD_NT
#define HCTR_GRAD_NT 1
#endif
typedef float f32x4 __attribute__((ext_vector_type(4)));
// A gradient row is read exactly once per step: it is loaded past the caches.  With sum-pooled bags (kPooled) a row
// is read once per key of its bag, so there it is loaded the ordinary way and the repeats hit the cache.
template <bool kPooled> __device__ __forceinline__ float4 grad_load(const float4 *p) {
  if (HCTR_GRAD_NT && !kPooled) {
    const f32x4 r = __builtin_nontemporal_load((const f32x4 *)p);
    return make_float4(r.x, r.y, r.z, r.w);
  }
  return *p;
}
template <bool kPooled> __device__ __forceinline__ float grad_load(const float *p) {
  if (HCTR_GRAD_NT && !kPooled) return __builtin_nontemporal_load(p);
  return *p;
}
// The gradient row of batch position `pos`: the position itself, or with sum-pooled bags of `bag` consecutive
// positions the row of the position's bag (every key of a bag receives the bag's gradient).
// kPooled is a compile-time switch: the plain push must not pay for the division in its load pipelines.
template <bool kPooled> __device__ __forceinline__ uint32_t grad_row(uint32_t pos, const BagDiv &bag) {
  return kPooled ? bag(pos) : pos;
}

template <int VEC> struct Vec;
template <> struct Vec<4> {
  typedef float4 T;
  static __device__ __forceinline__ T zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
  static __device__ __forceinline__ void add(T &a, const T &b) { a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; }
  static __device__ __forceinline__ T scale(const T &a, float s) { return make_float4(a.x * s, a.y * s, a.z * s, a.w * s); }
  // a store past the caches: for rows another shard's kernel reads next
  static __device__ __forceinline__ void store_away(T *p, const T &a) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    f4 v = {a.x, a.y, a.z, a.w};
    __builtin_nontemporal_store(v, (f4 *)p);
  }
};
template <> struct Vec<1> {
  typedef float T;
  static __device__ __forceinline__ T zero() { return 0.f; }
  static __device__ __forceinline__ void add(T &a, const T &b) { a += b; }
  static __device__ __forceinline__ T scale(const T &a, float s) { return a * s; }
  static __device__ __forceinline__ void store_away(T *p, const T &a) { __builtin_nontemporal_store(a, p); }
};

// The version / update counters of unique rank u and its entry among the pushed rows (gradient_index_kernel,
// generate_query.cu:51-83).  type: the update type of generate_query.cu:18-25; q: the row's place among the pushed rows.
template <typename K>
__device__ __forceinline__ void move_counters(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                              uint32_t u, slot_t o, int type, uint32_t q) {
  version_t cnt = (version_t)(p.run_start[u + 1] - p.run_start[u]);
  if (type == 1) t.ver[o] += cnt;
  else if (type >= 2) {
    version_t up = t.upd[o] + cnt;
    if (type == 2) {
      cnt = up;
      up = 0;
      t.ver[o] += cnt;
    }
    t.upd[o] = up;
  }
  if (type == 0 || type == 2) { // the rows the plan marks as pushed
    a.g_idx[q] = (index_t)(((const K *)p.ukey)[u] & (K)(((uint64_t)1 << id_bits) - 1));
    a.g_cnt[q] = cnt;
  }
}

// Applies the finished sum of unique rank u (already multiplied by -lr) to column(s) `col`.  Update types as in
// generate_query.cu:18-25.  The counters of the row move in the last blocks of the launch.
template <int VEC, typename K>
__device__ __forceinline__ void apply_row(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                          uint32_t u, typename Vec<VEC>::T s, uint32_t col) {
  typedef typename Vec<VEC>::T V;
  const slot_t o = p.uoff[u];
  const uint32_t W = t.width;
  if (t.nrank == 1) { // every key is owned and resident: type 1 only
    V *e = (V *)(t.emb + (size_t)o * W + col);
    V cur = *e;
    Vec<VEC>::add(cur, s);
    *e = cur;
    return;
  }
  const bool need = a.need[u] != 0;
  const int type = o == kNoSlot ? 0 : ((uint32_t)o >= t.n_cached ? 1 : (need ? 2 : 3));
  const uint32_t q = a.prefix[u];
  if (type != 0) {
    V *e = (V *)(t.emb + (size_t)o * W + col);
    V cur = *e;
    Vec<VEC>::add(cur, s);
    *e = cur;
  } else {
    Vec<VEC>::store_away((V *)(a.g_val + (size_t)q * W + col), s);
  }
  if (type >= 2) {
    V *g = (V *)(t.pend + (size_t)o * W + col);
    V pg = *g;
    Vec<VEC>::add(pg, s);
    if (type == 2) {
      Vec<VEC>::store_away((V *)(a.g_val + (size_t)q * W + col), pg);
      pg = Vec<VEC>::zero();
    }
    *g = pg;
  }
}

// ---- short role ----------------------------------------------------------------------------------------
// A group of LPR lanes owns kRunsPerGroup consecutive unique ranks and sums every run among them that is not
// long.  Everything the group needs first is requested before anything is waited for: the run bounds and
// resident offsets, then the destination rows, the first two gradient-row indices of every run and those
// gradient rows.  Nine runs out of ten are finished by that; longer ones continue eight rows at a time.
// Three runs per group: alone the kernel is 1 % faster with two, next to the index kernels of the following batch on the
// second stream it is 3 % faster with three (blocks that live longer lose less to what is scheduled beside them); from
// four on registers spill.
#ifndef HCTR_RUNS_PER_GROUP
#define HCTR_RUNS_PER_GROUP 3
#endif
constexpr int kRunsPerGroup = HCTR_RUNS_PER_GROUP;
constexpr int kHead = 2; // occurrences per run fetched up front
constexpr int kTail = 6; // occurrences per step after those

template <int VEC, int LPR, typename K, bool kSingle, bool kPooled>
__device__ __forceinline__ void short_role(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                           uint32_t block, uint32_t U) {
  typedef typename Vec<VEC>::T V;
  constexpr int G = kRunsPerGroup;
  constexpr int kGroups = kPushBlock / LPR;
  const uint32_t W = t.width, n = p.n;
  const uint32_t u0 = (block * kGroups + threadIdx.x / LPR) * G;
  if (u0 >= U) return;
  const uint32_t gl = threadIdx.x % LPR;
  const uint32_t *__restrict__ run_start = p.run_start;
  const uint32_t *__restrict__ sorted_arg = p.sorted_arg;
  const embed_t *__restrict__ grad = a.grad;
  uint32_t rs[G + 1];
  slot_t off[G];
#pragma unroll
  for (int i = 0; i <= G; i++) rs[i] = run_start[min(u0 + i, U)];
#pragma unroll
  for (int i = 0; i < G; i++) off[i] = p.uoff[min(u0 + i, U - 1)];
  // several shards: the update type of every run (generate_query.cu:18-25) and its place among the pushed rows
  int type[G];
  uint32_t q[G];
  if (!kSingle) {
    uint32_t nd[G];
#pragma unroll
    for (int i = 0; i < G; i++) {
      nd[i] = a.need[min(u0 + i, U - 1)];
      q[i] = a.prefix[min(u0 + i, U - 1)];
    }
#pragma unroll
    for (int i = 0; i < G; i++)
      type[i] = off[i] == kNoSlot ? 0 : ((uint32_t)off[i] >= t.n_cached ? 1 : (nd[i] ? 2 : 3));
  }
  const float neg_lr = t.neg_lr;

  for (uint32_t c0 = 0; c0 < W; c0 += LPR * VEC) {
    const uint32_t col = c0 + gl * VEC;
    const bool active = col < W;
    uint32_t len[G];
    bool mine[G];
    V e[G], pg[G];
    uint32_t si[G][kHead];
    V v[G][kHead];
#pragma unroll
    for (int i = 0; i < G; i++) {
      len[i] = rs[i + 1] - rs[i];
      mine[i] = u0 + i < U && len[i] <= kTinyRun && active;
    }
    // the rows the sums will be added to are requested before the gradient rows, not after the sums are done
#pragma unroll
    for (int i = 0; i < G; i++) {
      e[i] = Vec<VEC>::zero();
      if (mine[i] && (kSingle || type[i] != 0)) e[i] = *(const V *)(t.emb + (size_t)off[i] * W + col);
    }
    if (!kSingle) {
#pragma unroll
      for (int i = 0; i < G; i++) {
        pg[i] = Vec<VEC>::zero();
        if (mine[i] && type[i] >= 2) pg[i] = *(const V *)(t.pend + (size_t)off[i] * W + col);
      }
    }
#pragma unroll
    for (int i = 0; i < G; i++)
#pragma unroll
      for (int k = 0; k < kHead; k++) si[i][k] = grad_row<kPooled>(sorted_arg[min(rs[i] + k, n - 1)], a.bag);
#pragma unroll
    for (int i = 0; i < G; i++)
#pragma unroll
      for (int k = 0; k < kHead; k++) {
        v[i][k] = Vec<VEC>::zero();
        if (mine[i] && (uint32_t)k < len[i]) v[i][k] = grad_load<kPooled>((const V *)(grad + (size_t)si[i][k] * W + col));
      }
    V acc[G];
#pragma unroll
    for (int i = 0; i < G; i++) { // heads of all runs first: their registers are free before the tails start
      acc[i] = Vec<VEC>::zero();  // the reference starts every sum from 0
#pragma unroll
      for (int k = 0; k < kHead; k++)
        if (mine[i] && (uint32_t)k < len[i]) Vec<VEC>::add(acc[i], v[i][k]);
    }
#pragma unroll
    for (int i = 0; i < G; i++) {
      if (!mine[i]) continue;
      // the rest of the run (at most kTinyRun - kHead rows), in order, kTail rows at a time
      for (uint32_t j = rs[i] + kHead; j < rs[i + 1]; j += kTail) {
        uint32_t sj[kTail];
        V x[kTail];
#pragma unroll
        for (int k = 0; k < kTail; k++) sj[k] = grad_row<kPooled>(sorted_arg[min(j + k, rs[i + 1] - 1)], a.bag);
#pragma unroll
        for (int k = 0; k < kTail; k++) x[k] = grad_load<kPooled>((const V *)(grad + (size_t)sj[k] * W + col));
#pragma unroll
        for (int k = 0; k < kTail; k++)
          if (j + k < rs[i + 1]) Vec<VEC>::add(acc[i], x[k]);
      }
      const V scaled = Vec<VEC>::scale(acc[i], neg_lr);
      if (kSingle) {
        V r = e[i];
        Vec<VEC>::add(r, scaled);
        *(V *)(t.emb + (size_t)off[i] * W + col) = r; // the version counters move in the last blocks of the launch
      } else {
        // the same updates as apply_row(), with the rows already here
        if (type[i] != 0) {
          V r = e[i];
          Vec<VEC>::add(r, scaled);
          *(V *)(t.emb + (size_t)off[i] * W + col) = r;
        } else {
          Vec<VEC>::store_away((V *)(a.g_val + (size_t)q[i] * W + col), scaled);
        }
        if (type[i] >= 2) {
          V g = pg[i];
          Vec<VEC>::add(g, scaled);
          if (type[i] == 2) {
            Vec<VEC>::store_away((V *)(a.g_val + (size_t)q[i] * W + col), g);
            g = Vec<VEC>::zero();
          }
          *(V *)(t.pend + (size_t)off[i] * W + col) = g;
        }
      }
    }
  }
}

// ---- medium role ---------------------------------------------------------------------------------------
// Runs between kTinyRun and kLongRun occurrences: one group of LPR lanes per run of the list (groups stride
// over it).  The group first copies the run's gradient-row indices into LDS with one coalesced load, so that no
// later load waits for an index; then two batches of kBatch gradient rows are kept in flight while the rows are
// added in order.
template <int VEC, int LPR, typename K, bool kSingle, bool kPooled>
__device__ __forceinline__ void medium_role(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                            uint32_t *lds_idx, uint32_t block, uint32_t nblocks) {
  typedef typename Vec<VEC>::T V;
  constexpr int kGroups = kPushBlock / LPR;
  const uint32_t W = t.width;
  const uint32_t gl = threadIdx.x % LPR;
  uint32_t *my_idx = lds_idx + (threadIdx.x / LPR) * kLongRun; // this group's slice of the index staging area
  const uint32_t n_med = p.d_nlong[kMedCount];
  const uint32_t *__restrict__ sorted_arg = p.sorted_arg;
  const embed_t *__restrict__ grad = a.grad;
  const float neg_lr = t.neg_lr;
  for (uint32_t item = block * kGroups + threadIdx.x / LPR; item < n_med; item += nblocks * kGroups) {
    const uint32_t u = p.med_list[item];
    const uint32_t lo = p.run_start[u], hi = p.run_start[u + 1];
    const uint32_t len = hi - lo; // <= kLongRun
    const slot_t off = p.uoff[u];
    for (uint32_t q = gl; q < len; q += LPR) my_idx[q] = grad_row<kPooled>(sorted_arg[lo + q], a.bag);
    // a group never spans waves: the LDS writes above are ordered before the reads below in hardware; the
    // fence keeps the compiler from moving them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (uint32_t c0 = 0; c0 < W; c0 += LPR * VEC) {
      const uint32_t col = c0 + gl * VEC;
      const bool active = col < W;
      const embed_t *gcol = grad + (active ? col : 0);
      V e = Vec<VEC>::zero();
      if (kSingle && active) e = *(const V *)(t.emb + (size_t)off * W + col);
      V acc = Vec<VEC>::zero();
      V xa[kBatch], xb[kBatch];
      auto fetch = [&](V(&x)[kBatch], uint32_t q0) { // rows q0 .. q0+kBatch-1 of the run (clamped to its end)
#pragma unroll
        for (int k = 0; k < kBatch; k++) x[k] = grad_load<kPooled>((const V *)(gcol + (size_t)my_idx[min(q0 + k, len - 1)] * W));
      };
      auto add = [&](const V(&x)[kBatch], uint32_t q0) {
#pragma unroll
        for (int k = 0; k < kBatch; k++)
          if (q0 + k < len) Vec<VEC>::add(acc, x[k]);
      };
      fetch(xa, 0);
      for (uint32_t q = 0; q < len; q += 2 * kBatch) {
        if (q + kBatch < len) fetch(xb, q + kBatch);
        add(xa, q);
        if (q + 2 * kBatch < len) fetch(xa, q + 2 * kBatch);
        if (q + kBatch < len) add(xb, q + kBatch);
      }
      if (!active) continue;
      const V scaled = Vec<VEC>::scale(acc, neg_lr);
      if (kSingle) {
        Vec<VEC>::add(e, scaled);
        *(V *)(t.emb + (size_t)off * W + col) = e; // versions: bump_versions
      } else {
        apply_row<VEC, K>(t, id_bits, p, a, u, scaled, col);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier(); // the staging area is rewritten for the next run
  }
}

// ---- long role -----------------------------------------------------------------------------------------
// A block works on ONE column slice (CS columns) of a bundle of long runs at a time and treats the bundle as one
// stream of chunks, so that the loads of the next run are in flight while the current one is summed.  Runs are
// listed by length class, longest first; a bundle is 1..kTable runs of one class holding at least ~2048
// occurrences.  Tickets (bundle, slice) are handed out through one counter per group of blocks that share slices;
// the summing wave draws the next ticket and requests its run descriptors while the current bundle streams, so a
// change of bundle costs only the refill of the load pipeline.
// Wave 0 of the block only sums; the other 7 waves ("loaders") only move gradient rows global -> registers ->
// LDS ring.  A row slice is read by CS/VEC loader lanes; one block-wide load covers RPL = 448 / (CS/VEC)
// consecutive occurrences and a chunk is kRPT such loads (chunks never span two runs).  Loaders and the summing
// wave meet at one barrier per chunk: barrier m says "chunk m is in LDS".  A slot is overwritten kSlots
// barriers later, after the summing wave has passed the barrier that follows its reads.
constexpr int kLoaders = kPushBlock - kWave;
constexpr int kTable = 16;     // runs per bundle at most
#ifndef HCTR_SUM_BATCH
#define HCTR_SUM_BATCH 28
#endif
constexpr int kSumBatch = HCTR_SUM_BATCH; // rows the summing wave reads from LDS in one go (two such batches are live)

// the four floats of v to dst[0], dst[stride], dst[2 * stride], dst[3 * stride]
__device__ __forceinline__ void store_transposed(float *dst, uint32_t stride, const float4 &v) {
  dst[0] = v.x, dst[stride] = v.y, dst[2 * stride] = v.z, dst[3 * stride] = v.w;
}
__device__ __forceinline__ void store_transposed(float *, uint32_t, const float &) {} // generic path: never called

// a value that is the same in every lane, moved to a scalar register
__device__ __forceinline__ uint32_t uni(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// runs per bundle: classes halve in length -- one run of 2048 or more, 2 of 1024.., 4, 8, 16; `shrink` halves that
// (down to single runs) for batches with few long runs
__device__ __forceinline__ uint32_t bundle_runs(int cls, uint32_t shrink) {
  return cls <= 6 ? 1u : max(min(1u << (cls - 6), (uint32_t)kTable) >> shrink, 1u);
}

template <int VEC, typename K, int CSC, bool kPooled> // CSC: columns per slice if known at compile time, else 0
__device__ __forceinline__ void long_role(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                          float *lds, uint4 *table, uint32_t *shared, float *row_stash, int c_lo,
                                          int c_hi, uint32_t bidx, uint32_t nblk, uint32_t *counters) {
  typedef typename Vec<VEC>::T V;
  const uint32_t W = t.width;
  const uint32_t CS = CSC ? (uint32_t)CSC : min((uint32_t)kSlice, (W + VEC - 1) / VEC * VEC);
  uint32_t lanes = (CS + VEC - 1) / VEC; // loader lanes per row slice, rounded up to a power of two
  lanes = lanes <= 1 ? 1 : lanes <= 2 ? 2 : lanes <= 4 ? 4 : lanes <= 8 ? 8 : lanes <= 16 ? 16 : lanes <= 32 ? 32 : 64;
  const uint32_t RPL = CSC ? (uint32_t)(kLoaders / (CSC / VEC)) : kLoaders / lanes;
  const uint32_t CR = RPL * kRPT;                                   // rows per chunk
  constexpr int kChunkRows = CSC ? kRPT * (kLoaders / (CSC / VEC)) : 1; // CR as a constant on the fast path
  static_assert(!CSC || (kChunkRows % kSumBatch == 0 && kSumBatch % 4 == 0), "a chunk of the fast path is a whole number of sum batches");
  static_assert(!CSC || kSlots * CSC * (kChunkRows + 4) <= kSlots * kRPT * kPushBlock * VEC, "ring slots of the fast path fit the LDS area");
  const uint32_t slices = (W + CS - 1) / CS;
  // LDS layout of a ring slot.  Generic path: row-major [row][CS].  Fast path (CSC): column-major with the row
  // index fastest, [column place][pitch], pitch = rows + 4, so that the summing lane gets four consecutive rows of
  // its column with one 16-byte read; column c sits at place (c % 4) * (CSC / 4) + c / 4, which makes both the
  // loaders' 4-byte writes and the 16-byte reads free of bank conflicts (pitch % 8 == 4).
  const uint32_t pitch = CR + 4;
  const uint32_t slot_floats = CSC ? CS * pitch : CR * CS;
  const float neg_lr = t.neg_lr;
  const bool summer = threadIdx.x < kWave;
  const uint32_t lt = threadIdx.x - kWave; // loader thread number (meaningless on the summing wave)
  const uint32_t my_row = lt / lanes, my_lane = lt % lanes;
  const uint32_t *__restrict__ sorted_arg = p.sorted_arg;

  // tickets of this block's group: (bundle, slice) with the bundle changing slowest, so the longest runs go first
  const uint32_t share = min(min(slices, nblk), (uint32_t)kTicketLanes);
  const uint32_t lane_id = bidx % share;
  const uint32_t n_sl = (slices - lane_id + share - 1) / share; // slices lane_id, lane_id + share, ...
  const uint32_t group_blocks = (nblk - lane_id + share - 1) / share; // blocks drawing from this counter
  uint32_t cnt[kLongBuckets];
#pragma unroll
  for (int c = 0; c < kLongBuckets; c++) cnt[c] = (c >= c_lo && c < c_hi) ? uni(p.d_nlong[c]) : 0u;
  // A block streams a bundle at the pace its rows in flight allow (a few ns per occurrence), whatever the other
  // blocks do: a small batch, whose long runs make fewer tickets than there are blocks to draw them, gets smaller
  // bundles until every block has work or every bundle is a single run.  Every block computes the same value.
  uint32_t shrink = 0, nbundles;
  for (;;) {
    nbundles = 0;
#pragma unroll
    for (int c = 0; c < kLongBuckets; c++) nbundles += (cnt[c] + bundle_runs(c, shrink) - 1) / bundle_runs(c, shrink);
    if (shrink == 4 || nbundles * slices >= 2 * nblk) break;
    shrink++;
  }
  if (!nbundles) return;
  const uint32_t tickets = nbundles * n_sl;

  // summing wave: draws a ticket and requests the descriptors of its runs (one lane per run)
  uint4 pend = make_uint4(0, 0, 0, 0);
  uint32_t pend_runs = 0, pend_slice = 0;
  auto draw = [&]() {
    uint32_t tk = 0;
    if (threadIdx.x == 0) tk = atomicAdd(counters + lane_id, 1u);
    tk = (uint32_t)__builtin_amdgcn_readfirstlane((int)tk);
    pend_runs = 0;
    if (tk >= tickets) {
      // Every block of the group draws exactly one ticket past the end.  The block that draws the last of them
      // knows that nobody will touch the counter again in this launch and puts it back to zero, so that the same
      // batch can be pushed again (push_pull twice without a preprocess in between applies the gradient twice,
      // csrc/core/hetu_gpu_table.cu:9-41).
      if (threadIdx.x == 0 && tk == tickets + group_blocks - 1) atomicExch(counters + lane_id, 0u);
      return;
    }
    uint32_t bundle = tk / n_sl;
    pend_slice = lane_id + (tk % n_sl) * share;
    int cls = 0;
    uint32_t run0 = 0;
    bool found = false;
#pragma unroll
    for (int c = 0; c < kLongBuckets; c++) {
      const uint32_t bs = bundle_runs(c, shrink), nb = (cnt[c] + bs - 1) / bs;
      if (!found) {
        if (bundle < nb) {
          found = true;
          cls = c;
          run0 = bundle * bs;
          pend_runs = min(bs, cnt[c] - run0);
        } else {
          bundle -= nb;
        }
      }
    }
    if (threadIdx.x < pend_runs) pend = p.long_list[(size_t)cls * p.long_cap + run0 + threadIdx.x];
  };
  // ... and makes them the block's current bundle: descriptors, number of runs, chunks and the slice
  auto publish = [&]() {
    uint32_t chunks = threadIdx.x < pend_runs ? (pend.z + CR - 1) / CR : 0u;
    if (threadIdx.x < pend_runs) table[threadIdx.x] = pend; // rank, first position, length, offset
#pragma unroll
    for (int d = kTable / 2; d; d >>= 1) chunks += __shfl_down(chunks, d);
    if (threadIdx.x == 0) {
      shared[0] = pend_runs;
      shared[1] = chunks;
      shared[2] = pend_slice;
    }
  };

  if (summer) draw();
  for (;;) {
    if (summer) publish();
    __syncthreads();
    const uint32_t J = uni(shared[0]), G = uni(shared[1]), slice = uni(shared[2]); // runs, chunks and slice of this bundle
    if (!J) break;
    if (summer) draw(); // the requests stay in flight while this bundle streams

    if (!summer) {
      // ---------------- loaders ----------------
      const uint32_t lcol = my_lane * VEC; // column inside the slice
      const uint32_t col = slice * CS + lcol;
      const bool in_slice = lcol < CS && my_row < RPL;
      // Loads are unconditional and branch-free so that kDepth chunks stay in flight per thread: positions
      // past the end of a run re-read its last row (never summed), lanes outside the slice read column 0.
      const embed_t *gbase = a.grad + ((in_slice && col < W) ? col : 0);
      auto row_load = [&](uint32_t idx) -> V { return grad_load<kPooled>((const V *)(gbase + (size_t)idx * W)); };
      // cursor of the index stage, 2 * kDepth chunks ahead of the LDS stage; past the end of the stream it
      // stays on the last run
      uint32_t cj = 0, cc = 0;
      uint32_t clo, chi, cn;
      {
        const uint4 m = table[0];
        clo = uni(m.y);
        chi = clo + uni(m.z);
        cn = (uni(m.z) + CR - 1) / CR;
      }
      auto next_chunk = [&](uint32_t(&dst)[kRPT]) {
#pragma unroll
        for (int q = 0; q < kRPT; q++) dst[q] = grad_row<kPooled>(sorted_arg[min(clo + cc * CR + q * RPL + my_row, chi - 1)], a.bag);
        cc++;
        if (cc >= cn && cj + 1 < J) {
          cj++;
          const uint4 m = table[cj];
          clo = uni(m.y);
          chi = clo + uni(m.z);
          cn = (uni(m.z) + CR - 1) / CR;
          cc = 0;
        }
      };
      uint32_t idx[kDepth][kRPT];
      V val[kDepth][kRPT];
#pragma unroll
      for (int k = 0; k < kDepth; k++) next_chunk(idx[k]);
#pragma unroll
      for (int k = 0; k < kDepth; k++)
#pragma unroll
        for (int q = 0; q < kRPT; q++) val[k][q] = row_load(idx[k][q]);
#pragma unroll
      for (int k = 0; k < kDepth; k++) next_chunk(idx[k]);
      // invariant at step k of a round: val[k] holds chunk g0+k, idx[k] the row indices of chunk g0+k+kDepth
      uint32_t slot = 0;
      auto step = [&](int k) {
        float *sp = lds + slot * slot_floats;
        slot = slot + 1 == (uint32_t)kSlots ? 0 : slot + 1;
#pragma unroll
        for (int q = 0; q < kRPT; q++) {
          if (in_slice) {
            if (CSC) store_transposed(sp + my_lane * pitch + (q * RPL + my_row), (CSC / 4) * pitch, val[k][q]);
            else *(V *)(sp + (q * RPL + my_row) * CS + lcol) = val[k][q];
          }
          val[k][q] = row_load(idx[k][q]); // chunk + kDepth
        }
        next_chunk(idx[k]); // chunk + 2 * kDepth
        __syncthreads();    // barrier of this chunk
      };
      // Whole rounds run without a condition inside: with one, the compiler must assume that loads may have been
      // skipped and waits for nearly everything in flight before each use.
      uint32_t g0 = 0;
      for (; g0 + kDepth <= G; g0 += kDepth) {
#pragma unroll
        for (int k = 0; k < kDepth; k++) step(k);
      }
#pragma unroll
      for (int k = 0; k < kDepth; k++)
        if (g0 + k < G) step(k); // uniform over the block: the summing wave makes the same number of barriers
    } else {
      // ---------------- summing wave: one column per lane, rows strictly in order ----------------
      // the column this lane sums: lane = place in the fast path's layout
      const uint32_t mycol = slice * CS + (CSC ? (threadIdx.x % (CSC ? CSC / 4 : 1)) * 4 + threadIdx.x / (CSC ? CSC / 4 : 1) : threadIdx.x);
      const bool col_ok = threadIdx.x < CS && mycol < W;
      const bool direct = t.nrank == 1; // every key is owned and resident; the version counters move elsewhere
      uint32_t slot = 0;
      if (direct) {
        // The table rows the sums are added to, for every run of the bundle at once and parked in LDS: requested
        // run by run, each would arrive a memory round trip after its run had been summed (a run of a few hundred
        // occurrences is summed in a fraction of one), and the loaders would wait behind the full ring meanwhile.
        // This wait happens once per bundle, while the loaders' first rows are on their way.
        float rows[kTable];
#pragma unroll
        for (int j = 0; j < kTable; j++) {
          rows[j] = 0.f;
          if ((uint32_t)j < J && col_ok) rows[j] = t.emb[(size_t)table[j].w * W + mycol];
        }
#pragma unroll
        for (int j = 0; j < kTable; j++) row_stash[j * kWave + threadIdx.x] = rows[j];
      }
      for (uint32_t j = 0; j < J; j++) {
        const uint4 m = table[j];
        const uint32_t L = m.z;
        const uint32_t nfull = L / CR, nch = (L + CR - 1) / CR;
        float acc = 0.f; // the reference starts every sum from 0
        uint32_t c = 0;
        if (CSC) {
          // Full chunks, kSumBatch rows at a time, one batch ahead: the LDS reads of a batch are in flight while the
          // previous batch is added.  Reading the first batch of a chunk passes that chunk's barrier, i.e. the wave
          // is at most one barrier ahead of its adds, which the three ring slots allow.
          constexpr int kBatches = kChunkRows / kSumBatch; // per chunk, even
          static_assert(!CSC || kBatches % 2 == 0, "the two batch buffers alternate, a chunk starts on the first");
          const uint32_t lane_off = (threadIdx.x < CS ? threadIdx.x : 0) * pitch;
          const float *sp = lds;
          auto open_chunk = [&]() { // passes the chunk's barrier
            __syncthreads();
            sp = lds + slot * slot_floats + lane_off;
            slot = slot + 1 == (uint32_t)kSlots ? 0 : slot + 1;
          };
          auto read_batch = [&](int k, float(&dst)[kSumBatch]) { // batch k of the open chunk
            const float4 *bp = (const float4 *)(sp + k * kSumBatch);
#pragma unroll
            for (int q = 0; q < kSumBatch / 4; q++) {
              const float4 v = bp[q];
              dst[4 * q] = v.x, dst[4 * q + 1] = v.y, dst[4 * q + 2] = v.z, dst[4 * q + 3] = v.w;
            }
          };
          auto add_batch = [&](const float(&x)[kSumBatch]) {
#pragma unroll
            for (int q = 0; q < kSumBatch; q++) acc += x[q];
          };
          if (nfull) {
            float x0[kSumBatch], x1[kSumBatch];
            open_chunk();
            read_batch(0, x0);
            // all chunks but the last: straight-line code, so that the waits for LDS data stay exact
            for (uint32_t cc2 = 0; cc2 + 1 < nfull; cc2++) {
#pragma unroll
              for (int k = 0; k < kBatches; k += 2) {
                read_batch(k + 1, x1);
                add_batch(x0);
                if (k + 2 < kBatches) {
                  read_batch(k + 2, x0);
                } else {
                  open_chunk();
                  read_batch(0, x0);
                }
                add_batch(x1);
              }
            }
#pragma unroll
            for (int k = 0; k < kBatches; k += 2) { // the last full chunk
              read_batch(k + 1, x1);
              add_batch(x0);
              if (k + 2 < kBatches) read_batch(k + 2, x0);
              add_batch(x1);
            }
          }
          c = nfull;
        }
        for (; c < nch; c++) { // generic path, and the partial last chunk of the fast path
          __syncthreads();     // barrier of this chunk
          const uint32_t rstride = CSC ? 1u : CS; // distance between two rows of this lane's column
          const float *col_ptr = lds + slot * slot_floats + threadIdx.x * (CSC ? pitch : 1u);
          slot = slot + 1 == (uint32_t)kSlots ? 0 : slot + 1;
          if (threadIdx.x < CS) {
            const uint32_t rows = min(CR, L - c * CR);
            uint32_t r = 0;
            for (; r + 8 <= rows; r += 8) {
              float x[8];
#pragma unroll
              for (int q = 0; q < 8; q++) x[q] = col_ptr[(r + q) * rstride];
#pragma unroll
              for (int q = 0; q < 8; q++) acc += x[q];
            }
            for (; r < rows; r++) acc += col_ptr[r * rstride];
          }
        }
        if (col_ok) {
          const float scaled = acc * neg_lr;
          if (direct) t.emb[(size_t)m.w * W + mycol] = row_stash[j * kWave + threadIdx.x] + scaled;
          else apply_row<1, K>(t, id_bits, p, a, m.x, scaled, mycol);
        }
      }
    }
    __syncthreads(); // everybody is done with the table and the ring
  }
}

// all roles in one launch: the long chains start first, medium and short blocks fill the machine behind them, the
// version counters of a single shard come last
template <int VEC, int LPR, typename K, bool kSingle, bool kPooled>
#ifndef HCTR_PUSH_WAVES
#define HCTR_PUSH_WAVES 4
#endif
__global__ __launch_bounds__(kPushBlock) __attribute__((amdgpu_waves_per_eu(HCTR_PUSH_WAVES, 8))) void push_fused(TableView t, int id_bits, BatchView p, PushArgs a, uint32_t U) {
  // one LDS area for whichever role the block plays: the row ring of the long role or the index staging of the
  // medium role (one slice of kLongRun indices per group)
  constexpr int kRingWords = kSlots * kRPT * kPushBlock * VEC;
  constexpr int kStageWords = (kPushBlock / LPR) * (int)kLongRun;
  __shared__ __align__(16) float lds[kRingWords > kStageWords ? kRingWords : kStageWords];
  __shared__ uint4 run_table[kTable];
  __shared__ uint32_t run_totals[3];
  __shared__ float row_stash[kTable * kWave]; // long role: the table rows of a bundle's runs (one slice, one lane each)
  if (blockIdx.x < kLongBlocks) {
    // Every block first takes tickets of the longest runs, which are cut into narrower column slices so that more
    // blocks feed each of them (the blocks of a saturated memory system get equal shares of it, and a chain
    // advances with the share of the block that feeds it), then tickets of the other long runs.
    uint32_t *tk = p.d_nlong + kTicketBase;
    if (VEC == 4 && t.width % kSlice == 0) {
      long_role<VEC, K, (VEC == 4 ? kGiantSlice : 0), kPooled>(t, id_bits, p, a, lds, run_table, run_totals, row_stash, 0, kGiantClasses,
                                                      blockIdx.x, kLongBlocks, tk);
      long_role<VEC, K, (VEC == 4 ? kSlice : 0), kPooled>(t, id_bits, p, a, lds, run_table, run_totals, row_stash, kGiantClasses, kLongBuckets,
                                                 blockIdx.x, kLongBlocks, tk + kTicketLanes);
    } else {
      long_role<VEC, K, 0, kPooled>(t, id_bits, p, a, lds, run_table, run_totals, row_stash, 0, kLongBuckets, blockIdx.x, kLongBlocks, tk);
    }
  } else if (blockIdx.x < kLongBlocks + kMedBlocks) { // medium runs take long per block: they start early
    medium_role<VEC, LPR, K, kSingle, kPooled>(t, id_bits, p, a, (uint32_t *)lds, blockIdx.x - kLongBlocks, kMedBlocks);
  } else {
    constexpr int kGroups = kPushBlock / LPR;
    const uint32_t short_blocks = div_up_dev(U, kGroups * kRunsPerGroup);
    const uint32_t b = blockIdx.x - kLongBlocks - kMedBlocks;
    if (b < short_blocks) {
      short_role<VEC, LPR, K, kSingle, kPooled>(t, id_bits, p, a, b, U);
    } else {
      // The counters of every unique key, one thread per key, in the last blocks of the grid: they depend on the
      // batch's index and plan only, not on the sums.
      const uint32_t u = (b - short_blocks) * kPushBlock + threadIdx.x;
      if (u < U) {
        if (kSingle) {
          // Single shard: every key is owned, so the only counter is the row version, which grows by the number of
          // duplicates (generate_query.cu:68-69).  Nontemporal: a counter line is touched once per step; left in the
          // cache it is written back in the middle of the gather that follows.
          version_t *vp = &t.ver[p.uoff[u]];
          const version_t v = __builtin_nontemporal_load(vp) + (version_t)(p.run_start[u + 1] - p.run_start[u]);
          __builtin_nontemporal_store(v, vp);
        } else {
          const slot_t o = p.uoff[u];
          const bool need = a.need[u] != 0;
          const int type = o == kNoSlot ? 0 : ((uint32_t)o >= t.n_cached ? 1 : (need ? 2 : 3));
          move_counters<K>(t, id_bits, p, a, u, o, type, a.prefix[u]);
        }
      }
    }
  }
}

template <typename K>
__global__ __launch_bounds__(256) void place_rows(const K *__restrict__ ukey, uint32_t U, int id_bits,
                                                  const uint32_t *__restrict__ prefix,
                                                  const uint32_t *__restrict__ delta, uint32_t *__restrict__ pos) {
  const uint32_t u = blockIdx.x * 256 + threadIdx.x;
  if (u < U) pos[u] = prefix[u] + delta[(uint32_t)(ukey[u] >> id_bits)];
}

template <int VEC, int LPR, typename K, bool kSingle, bool kPooled>
void launch_push_t(hipStream_t st, const TableView &t, int id_bits, const BatchView &p, uint32_t U, const PushArgs &a) {
  constexpr int kGroups = kPushBlock / LPR;
  const unsigned ver_blocks = div_up(U, kPushBlock); // the counters of every unique key
  const unsigned rest = kMedBlocks + div_up(U, kGroups * kRunsPerGroup) + ver_blocks;
  hipLaunchKernelGGL((push_fused<VEC, LPR, K, kSingle, kPooled>), dim3(kLongBlocks + rest), dim3(kPushBlock), 0, st, t, id_bits, p,
                     a, U);
}

template <int VEC, typename K, bool kSingle, bool kPooled>
void launch_push_p(hipStream_t ps, const TableView &t, int id_bits, const BatchView &p, uint32_t U,
                   const PushArgs &a) {
  const uint32_t lanes = (t.width + VEC - 1) / VEC;
  if (lanes <= 4) launch_push_t<VEC, 4, K, kSingle, kPooled>(ps, t, id_bits, p, U, a);
  else if (lanes <= 8) launch_push_t<VEC, 8, K, kSingle, kPooled>(ps, t, id_bits, p, U, a);
  else if (lanes <= 16) launch_push_t<VEC, 16, K, kSingle, kPooled>(ps, t, id_bits, p, U, a);
  else if (lanes <= 32) launch_push_t<VEC, 32, K, kSingle, kPooled>(ps, t, id_bits, p, U, a);
  else launch_push_t<VEC, 64, K, kSingle, kPooled>(ps, t, id_bits, p, U, a);
}

template <int VEC, typename K, bool kSingle>
void launch_push_v(hipStream_t ps, const TableView &t, int id_bits, const BatchView &p, uint32_t U,
                   const PushArgs &a) {
  if (a.bag.bag > 1) launch_push_p<VEC, K, kSingle, true>(ps, t, id_bits, p, U, a);
  else launch_push_p<VEC, K, kSingle, false>(ps, t, id_bits, p, U, a);
}

template <int VEC, typename K>
void launch_push_k(hipStream_t ps, const TableView &t, int id_bits, const BatchView &p, uint32_t U,
                   const PushArgs &a) {
  if (t.nrank == 1) launch_push_v<VEC, K, true>(ps, t, id_bits, p, U, a);
  else launch_push_v<VEC, K, false>(ps, t, id_bits, p, U, a);
}

} // namespace

void launch_place_rows(hipStream_t s, const KeyLayout &kl, const BatchView &prev, uint32_t n_unique,
                       const uint32_t *prefix, const uint32_t *delta, uint32_t *pos) {
  if (!n_unique) return;
  if (kl.wide)
    hipLaunchKernelGGL(place_rows<uint64_t>, dim3(div_up(n_unique, 256)), dim3(256), 0, s, (const uint64_t *)prev.ukey,
                       n_unique, kl.id_bits, prefix, delta, pos);
  else
    hipLaunchKernelGGL(place_rows<uint32_t>, dim3(div_up(n_unique, 256)), dim3(256), 0, s, (const uint32_t *)prev.ukey,
                       n_unique, kl.id_bits, prefix, delta, pos);
  HCTR_HIP(hipGetLastError());
}

void launch_push(hipStream_t ps, const TableView &t, const KeyLayout &kl, const BatchView &prev, uint32_t n_unique,
                 const PushArgs &a) {
  if (!prev.n || !n_unique) return;
  const bool vec4 = t.width % 4 == 0 && ((uintptr_t)a.grad % 16) == 0;
  if (vec4) {
    if (kl.wide) launch_push_k<4, uint64_t>(ps, t, kl.id_bits, prev, n_unique, a);
    else launch_push_k<4, uint32_t>(ps, t, kl.id_bits, prev, n_unique, a);
  } else {
    if (kl.wide) launch_push_k<1, uint64_t>(ps, t, kl.id_bits, prev, n_unique, a);
    else launch_push_k<1, uint32_t>(ps, t, kl.id_bits, prev, n_unique, a);
  }
  HCTR_HIP(hipGetLastError());
}

} // namespace hctr
