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
//
// One launch, two roles (block index decides):
//  * long role (first blocks): a run longer than kLongRun is streamed by a whole block.  All 512 threads
//    keep kDepth 16-byte loads of gradient rows in flight each and stage them through a ring of LDS slots;
//    the first wave adds the staged rows in order, one column per lane.  The serial chain costs one LDS read
//    and one add per duplicate while the memory latency is covered by the whole block.  A run is split by
//    column slices of kSlice floats over several blocks.
//  * tile role: the sorted occurrence list is cut into tiles of kTileOcc occurrences; a group of LPR lanes
//    (LPR*VEC floats = one row) sums the short runs that START in its tile, walking past the tile end to
//    finish the last one.  Occurrences of long runs are flagged in rank_sorted and skipped.
#include "kernels.h"

namespace hctr {

// tuning knobs (overridable at compile time for experiments)
#ifndef HCTR_TILE_BATCH
#define HCTR_TILE_BATCH 8
#endif
#ifndef HCTR_DEPTH
#define HCTR_DEPTH 8
#endif
#ifndef HCTR_SLICE
#define HCTR_SLICE 64
#endif
#ifndef HCTR_LONG_BLOCKS
#define HCTR_LONG_BLOCKS 1024
#endif
#ifndef HCTR_ONLY_ROLE
#define HCTR_ONLY_ROLE 0 // 1: long role only, 2: tile role only (timing experiments; results are incomplete)
#endif
constexpr int kTileOcc = 32;
constexpr int kPushBlock = 512;
constexpr int kBatch = HCTR_TILE_BATCH;   // tile role: gradient rows in flight per group
constexpr int kDepth = HCTR_DEPTH;        // long role: loads in flight per thread
constexpr int kSlots = 4;                 // long role: LDS ring slots
constexpr int kSlice = HCTR_SLICE;        // long role: columns per block
constexpr int kLongBlocks = HCTR_LONG_BLOCKS;

size_t push_tiles(uint32_t n_prev) { return (n_prev + kTileOcc - 1) / kTileOcc; }

namespace {

template <int VEC> struct Vec;
template <> struct Vec<4> {
  typedef float4 T;
  static __device__ __forceinline__ T zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
  static __device__ __forceinline__ void add(T &a, const T &b) { a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; }
  static __device__ __forceinline__ T scale(const T &a, float s) { return make_float4(a.x * s, a.y * s, a.z * s, a.w * s); }
};
template <> struct Vec<1> {
  typedef float T;
  static __device__ __forceinline__ T zero() { return 0.f; }
  static __device__ __forceinline__ void add(T &a, const T &b) { a += b; }
  static __device__ __forceinline__ T scale(const T &a, float s) { return a * s; }
};

// Applies the finished sum of unique rank u (already multiplied by -lr) to column(s) `col`.
// `counters`: this lane also moves the version / update counters.  Update types as in generate_query.cu:18-25.
template <int VEC, typename K>
__device__ __forceinline__ void apply_row(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                          uint32_t u, typename Vec<VEC>::T s, uint32_t col, bool counters) {
  typedef typename Vec<VEC>::T V;
  const slot_t o = p.uoff[u];
  const uint32_t W = t.width;
  if (t.nrank == 1) { // every key is owned and resident: type 1 only
    V *e = (V *)(t.emb + (size_t)o * W + col);
    V cur = *e;
    Vec<VEC>::add(cur, s);
    *e = cur;
    if (counters) t.ver[o] += (version_t)(p.run_start[u + 1] - p.run_start[u]);
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
    *(V *)(a.g_val + (size_t)q * W + col) = s;
  }
  if (type >= 2) {
    V *g = (V *)(t.pend + (size_t)o * W + col);
    V pg = *g;
    Vec<VEC>::add(pg, s);
    if (type == 2) {
      *(V *)(a.g_val + (size_t)q * W + col) = pg;
      pg = Vec<VEC>::zero();
    }
    *g = pg;
  }
  if (counters) { // gradient_index_kernel, generate_query.cu:51-83
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
    if (need) {
      a.g_idx[q] = (index_t)(((const K *)p.ukey)[u] & (K)(((uint64_t)1 << id_bits) - 1));
      a.g_cnt[q] = cnt;
    }
  }
}

// ---- tile role -----------------------------------------------------------------------------------------
template <int VEC, int LPR, typename K>
__device__ __forceinline__ void tile_role(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                          uint32_t block) {
  typedef typename Vec<VEC>::T V;
  constexpr int kGroups = kPushBlock / LPR;
  const uint32_t n = p.n, W = t.width;
  const uint32_t tile = block * kGroups + threadIdx.x / LPR;
  const uint32_t gl = threadIdx.x % LPR;
  const uint32_t j0 = tile * kTileOcc;
  if (j0 >= n) return;
  const uint32_t j1 = min(j0 + kTileOcc, n);
  // a run that started before the tile belongs to the group of an earlier tile (or to the long role)
  const uint32_t head = p.rank_sorted[j0];
  const bool head_foreign = j0 > 0 && p.rank_sorted[j0 - 1] == head;
  // the last run of the tile is finished past the tile end if it is short and continues
  uint32_t je = j1;
  {
    const uint32_t ul = p.rank_sorted[j1 - 1];
    if (!(ul & kLongFlag) && j1 < n && p.rank_sorted[j1] == ul && !(head_foreign && ul == head))
      je = p.run_start[ul + 1];
  }
  const float neg_lr = t.neg_lr;

  for (uint32_t c0 = 0; c0 < W; c0 += LPR * VEC) {
    const uint32_t col = c0 + gl * VEC;
    const bool active = col < W;
    V acc = Vec<VEC>::zero();
    uint32_t cur_u = 0;
    bool have = false;
    for (uint32_t j = j0; j < je; j += kBatch) {
      uint32_t su[kBatch], ru[kBatch];
      bool use[kBatch];
      V v[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; k++) {
        const bool ok = j + k < je;
        su[k] = ok ? p.sorted_arg[j + k] : 0u;
        ru[k] = ok ? p.rank_sorted[j + k] : kLongFlag;
      }
#pragma unroll
      for (int k = 0; k < kBatch; k++) {
        use[k] = !(ru[k] & kLongFlag) && !(head_foreign && ru[k] == head);
        v[k] = Vec<VEC>::zero();
        if (use[k] && active) v[k] = *(const V *)(a.grad + (size_t)su[k] * W + col);
      }
#pragma unroll
      for (int k = 0; k < kBatch; k++) {
        if (!use[k]) continue;
        if (have && ru[k] != cur_u) {
          if (active) apply_row<VEC, K>(t, id_bits, p, a, cur_u, Vec<VEC>::scale(acc, neg_lr), col, c0 == 0 && gl == 0);
          acc = Vec<VEC>::zero();
        }
        cur_u = ru[k];
        have = true;
        Vec<VEC>::add(acc, v[k]);
      }
    }
    if (have && active) apply_row<VEC, K>(t, id_bits, p, a, cur_u, Vec<VEC>::scale(acc, neg_lr), col, c0 == 0 && gl == 0);
  }
}

// ---- long role -----------------------------------------------------------------------------------------
// Work item = (long run, column slice of CS columns).  Wave 0 of the block only sums; the other 7 waves
// ("loaders") only move gradient rows global -> registers -> LDS ring.  A row slice is read by CS/VEC loader
// lanes, so one block-wide load covers RPL = 448 / (CS/VEC) consecutive occurrences ("chunk").
// Loaders and the summing wave meet at one barrier per chunk: barrier m says "chunk m is in LDS".
constexpr int kLoaders = kPushBlock - kWave;

template <int VEC, typename K, int CSC> // CSC: columns per slice if known at compile time (64), else 0
__device__ __forceinline__ void long_role(const TableView &t, int id_bits, const BatchView &p, const PushArgs &a,
                                          uint32_t first_item, float *lds) {
  typedef typename Vec<VEC>::T V;
  const uint32_t W = t.width;
  const uint32_t CS = CSC ? (uint32_t)CSC : min((uint32_t)kSlice, (W + VEC - 1) / VEC * VEC);
  uint32_t lanes = (CS + VEC - 1) / VEC; // loader lanes per row slice, rounded up to a power of two
  lanes = lanes <= 1 ? 1 : lanes <= 2 ? 2 : lanes <= 4 ? 4 : lanes <= 8 ? 8 : lanes <= 16 ? 16 : lanes <= 32 ? 32 : 64;
  const uint32_t RPL = CSC ? (uint32_t)(kLoaders / (CSC / VEC)) : kLoaders / lanes;
  constexpr int kRows = CSC ? kLoaders / (CSC / VEC) : 1; // RPL as a constant on the fast path
  const uint32_t slices = (W + CS - 1) / CS;
  const uint32_t slot_floats = RPL * CS;
  const uint32_t items = *p.d_nlong * slices;
  const float neg_lr = t.neg_lr;
  const bool summer = threadIdx.x < kWave;
  const uint32_t lt = threadIdx.x - kWave; // loader thread number (meaningless on the summing wave)
  const uint32_t my_row = lt / lanes, my_lane = lt % lanes;

  for (uint32_t item = first_item; item < items; item += kLongBlocks) {
    const uint32_t u = p.long_list[item / slices];
    const uint32_t slice = item % slices;
    const uint32_t lo = p.run_start[u], hi = p.run_start[u + 1];
    const uint32_t L = hi - lo;
    const uint32_t nchunks = (L + RPL - 1) / RPL;
    if (!summer) {
      // ---------------- loaders ----------------
      const uint32_t lcol = my_lane * VEC; // column inside the slice
      const uint32_t col = slice * CS + lcol;
      const bool in_slice = lcol < CS && my_row < RPL;
      // Loads are unconditional and branch-free so that kDepth of them stay in flight per thread: positions
      // past the end of the run re-read its last row (never summed), lanes outside the slice read column 0.
      const embed_t *gbase = a.grad + ((in_slice && col < W) ? col : 0);
      auto row_index = [&](uint32_t c) -> uint32_t { return p.sorted_arg[min(lo + c * RPL + my_row, hi - 1)]; };
      auto row_load = [&](uint32_t idx) -> V { return *(const V *)(gbase + (size_t)idx * W); };
      uint32_t idx_a[kDepth], idx_b[kDepth];
      V val[kDepth];
#pragma unroll
      for (int k = 0; k < kDepth; k++) idx_a[k] = row_index(k);
#pragma unroll
      for (int k = 0; k < kDepth; k++) idx_b[k] = row_index(kDepth + k);
#pragma unroll
      for (int k = 0; k < kDepth; k++) val[k] = row_load(idx_a[k]);
      // invariant at the top of a round: val[k] holds chunk c0+k, idx_b[k] the row index of chunk c0+kDepth+k
      for (uint32_t c0 = 0; c0 < nchunks; c0 += kDepth) {
#pragma unroll
        for (int k = 0; k < kDepth; k++) idx_a[k] = idx_b[k];
#pragma unroll
        for (int k = 0; k < kDepth; k++) idx_b[k] = row_index(c0 + 2 * kDepth + k);
#pragma unroll
        for (int k = 0; k < kDepth; k++) {
          const uint32_t c = c0 + k;
          if (c < nchunks) { // uniform over the block: the summing wave makes the same number of barriers
            float *slot = lds + (c % kSlots) * slot_floats;
            if (in_slice) *(V *)(slot + my_row * CS + lcol) = val[k];
            val[k] = row_load(idx_a[k]); // chunk c + kDepth
            __syncthreads();             // barrier c
          }
        }
      }
    } else {
      // ---------------- summing wave: one column per lane, rows strictly in order ----------------
      float acc = 0.f;
      const uint32_t nfull = L / RPL; // chunks with all RPL rows
      uint32_t c = 0;
      if (CSC) {
        // software pipeline: the LDS reads of chunk c+1 are issued before the adds of chunk c
        float xa[kRows], xb[kRows];
        if (nfull > 0) {
          __syncthreads(); // barrier 0
          const float *sp = lds + threadIdx.x;
#pragma unroll
          for (int q = 0; q < kRows; q++) xa[q] = sp[q * CSC];
          for (c = 1; c + 1 < nfull; c += 2) {
            __syncthreads(); // barrier c
            const float *s1 = lds + (c % kSlots) * slot_floats + threadIdx.x;
#pragma unroll
            for (int q = 0; q < kRows; q++) xb[q] = s1[q * CSC];
#pragma unroll
            for (int q = 0; q < kRows; q++) acc += xa[q];
            __syncthreads(); // barrier c + 1
            const float *s2 = lds + ((c + 1) % kSlots) * slot_floats + threadIdx.x;
#pragma unroll
            for (int q = 0; q < kRows; q++) xa[q] = s2[q * CSC];
#pragma unroll
            for (int q = 0; q < kRows; q++) acc += xb[q];
          }
          if (c < nfull) { // one more full chunk
            __syncthreads(); // barrier c
            const float *s1 = lds + (c % kSlots) * slot_floats + threadIdx.x;
#pragma unroll
            for (int q = 0; q < kRows; q++) xb[q] = s1[q * CSC];
#pragma unroll
            for (int q = 0; q < kRows; q++) acc += xa[q];
#pragma unroll
            for (int q = 0; q < kRows; q++) acc += xb[q];
            c++;
          } else {
#pragma unroll
            for (int q = 0; q < kRows; q++) acc += xa[q];
          }
        }
      }
      for (; c < nchunks; c++) { // generic path, and the partial last chunk of the fast path
        __syncthreads();         // barrier c
        if (threadIdx.x < CS) {
          const float *col_ptr = lds + (c % kSlots) * slot_floats + threadIdx.x;
          const uint32_t rows = min(RPL, L - c * RPL);
          uint32_t r = 0;
          for (; r + 8 <= rows; r += 8) {
            float x[8];
#pragma unroll
            for (int q = 0; q < 8; q++) x[q] = col_ptr[(r + q) * CS];
#pragma unroll
            for (int q = 0; q < 8; q++) acc += x[q];
          }
          for (; r < rows; r++) acc += col_ptr[r * CS];
        }
      }
      if (threadIdx.x < CS && slice * CS + threadIdx.x < W)
        apply_row<1, K>(t, id_bits, p, a, u, acc * neg_lr, slice * CS + threadIdx.x, slice == 0 && threadIdx.x == 0);
    }
    __syncthreads(); // the ring is reused by the next item
  }
}

template <int VEC, int LPR, typename K>
__global__ __launch_bounds__(kPushBlock) void segment_sum_apply(TableView t, int id_bits, BatchView p, PushArgs a) {
  __shared__ __align__(16) float lds[kSlots * kPushBlock * VEC];
  if (blockIdx.x < kLongBlocks) {
    if (HCTR_ONLY_ROLE != 2) {
      if (VEC == 4 && t.width % 64 == 0) long_role<VEC, K, (VEC == 4 ? 64 : 0)>(t, id_bits, p, a, blockIdx.x, lds);
      else long_role<VEC, K, 0>(t, id_bits, p, a, blockIdx.x, lds);
    }
  } else {
    if (HCTR_ONLY_ROLE != 1) tile_role<VEC, LPR, K>(t, id_bits, p, a, blockIdx.x - kLongBlocks);
  }
}

template <int VEC, int LPR, typename K>
void launch_push_t(hipStream_t s, const TableView &t, int id_bits, const BatchView &p, const PushArgs &a) {
  constexpr int kGroups = kPushBlock / LPR;
  const unsigned tiles = (unsigned)push_tiles(p.n);
  hipLaunchKernelGGL((segment_sum_apply<VEC, LPR, K>), dim3(kLongBlocks + div_up(tiles, kGroups)), dim3(kPushBlock),
                     0, s, t, id_bits, p, a);
}

template <int VEC, typename K>
void launch_push_v(hipStream_t s, const TableView &t, int id_bits, const BatchView &p, const PushArgs &a) {
  const uint32_t lanes = (t.width + VEC - 1) / VEC;
  if (lanes <= 4) launch_push_t<VEC, 4, K>(s, t, id_bits, p, a);
  else if (lanes <= 8) launch_push_t<VEC, 8, K>(s, t, id_bits, p, a);
  else if (lanes <= 16) launch_push_t<VEC, 16, K>(s, t, id_bits, p, a);
  else if (lanes <= 32) launch_push_t<VEC, 32, K>(s, t, id_bits, p, a);
  else launch_push_t<VEC, 64, K>(s, t, id_bits, p, a);
}

} // namespace

void launch_push(hipStream_t s, const TableView &t, const KeyLayout &kl, const BatchView &prev, const PushArgs &a) {
  if (!prev.n) return;
  const bool vec4 = t.width % 4 == 0 && ((uintptr_t)a.grad % 16) == 0;
  if (vec4) {
    if (kl.wide) launch_push_v<4, uint64_t>(s, t, kl.id_bits, prev, a);
    else launch_push_v<4, uint32_t>(s, t, kl.id_bits, prev, a);
  } else {
    if (kl.wide) launch_push_v<1, uint64_t>(s, t, kl.id_bits, prev, a);
    else launch_push_v<1, uint32_t>(s, t, kl.id_bits, prev, a);
  }
  HCTR_HIP(hipGetLastError());
}

} // namespace hctr
