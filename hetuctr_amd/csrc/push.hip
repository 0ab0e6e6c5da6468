// Gradient push: deterministic segment-sum of the gradient rows of every unique key of the previous
// batch, fused with the SGD write-back to the table, the hot-row cache, the pending-gradient store,
// the version / update counters and the push buffer.
// Reference: csrc/core/generate_query.cu:8-89 (gradient_reduction_kernel, gradient_index_kernel).
//
// Summation order: the reference adds the gradient rows of one key serially, in ascending batch position,
// then multiplies once by -lr and adds once to the row.  fp32 addition is not associative, so any other
// order differs from it in the last bits by an amount that grows with the number of duplicates.  Here
// every run of equal keys is summed by ONE group of lanes, in exactly that order: sums are bit-identical
// to the reference's order (compiled without fused multiply-add contraction), for any skew.
//
// Work decomposition: the sorted occurrence list is cut into tiles of kTileOcc consecutive occurrences; a
// group of LPR lanes (LPR*VEC floats = one row, or a 256-float chunk of it) owns the runs that START in
// its tile.  It skips the head of the tile if that belongs to a run started earlier, and walks past the
// end of its tile to finish its last run.
#include "kernels.h"

namespace hctr {

constexpr int kTileOcc = 32;
constexpr int kPushBlock = 256;
constexpr int kBatch = 8; // gradient rows in flight per group

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
// `first_chunk` lane 0 also moves the counters.  Update types as in generate_query.cu:18-25.
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

// grid.x covers the tiles, kPushBlock/LPR groups per block.
template <int VEC, int LPR, typename K>
__global__ __launch_bounds__(kPushBlock) void segment_sum_apply(TableView t, int id_bits, BatchView p, PushArgs a) {
  typedef typename Vec<VEC>::T V;
  constexpr int kGroups = kPushBlock / LPR;
  const uint32_t n = p.n, W = t.width;
  const uint32_t tile = blockIdx.x * kGroups + threadIdx.x / LPR;
  const uint32_t gl = threadIdx.x % LPR;
  const uint32_t j0 = tile * kTileOcc;
  if (j0 >= n) return;
  const uint32_t j1 = min(j0 + kTileOcc, n);
  // runs that start in [j0, j1) are this group's; [jb, je) is the span of occurrences it sums
  uint32_t jb = j0;
  {
    const uint32_t u0 = p.rank_sorted[j0];
    if (j0 > 0 && p.rank_sorted[j0 - 1] == u0) jb = p.run_start[u0 + 1];
  }
  if (jb >= j1) return;
  uint32_t je = j1;
  {
    const uint32_t ul = p.rank_sorted[j1 - 1];
    if (j1 < n && p.rank_sorted[j1] == ul) je = p.run_start[ul + 1];
  }
  const float neg_lr = t.neg_lr;

  for (uint32_t c0 = 0; c0 < W; c0 += LPR * VEC) {
    const uint32_t col = c0 + gl * VEC;
    const bool active = col < W;
    V acc = Vec<VEC>::zero();
    uint32_t cur_u = p.rank_sorted[jb];
    for (uint32_t j = jb; j < je; j += kBatch) {
      uint32_t su[kBatch], ru[kBatch];
      V v[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; k++) {
        const bool ok = j + k < je;
        su[k] = ok ? p.sorted_arg[j + k] : 0u;
        ru[k] = ok ? p.rank_sorted[j + k] : 0xffffffffu;
      }
#pragma unroll
      for (int k = 0; k < kBatch; k++) {
        v[k] = Vec<VEC>::zero();
        if (j + k < je && active) v[k] = *(const V *)(a.grad + (size_t)su[k] * W + col);
      }
#pragma unroll
      for (int k = 0; k < kBatch; k++) {
        if (j + k >= je) break;
        if (ru[k] != cur_u) {
          if (active) apply_row<VEC, K>(t, id_bits, p, a, cur_u, Vec<VEC>::scale(acc, neg_lr), col, c0 == 0 && gl == 0);
          acc = Vec<VEC>::zero();
          cur_u = ru[k];
        }
        Vec<VEC>::add(acc, v[k]);
      }
    }
    if (active) apply_row<VEC, K>(t, id_bits, p, a, cur_u, Vec<VEC>::scale(acc, neg_lr), col, c0 == 0 && gl == 0);
  }
}

template <int VEC, int LPR, typename K>
void launch_push_t(hipStream_t s, const TableView &t, int id_bits, const BatchView &p, const PushArgs &a) {
  constexpr int kGroups = kPushBlock / LPR;
  const unsigned tiles = (unsigned)push_tiles(p.n);
  hipLaunchKernelGGL((segment_sum_apply<VEC, LPR, K>), dim3(div_up(tiles, kGroups)), dim3(kPushBlock), 0, s, t,
                     id_bits, p, a);
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
