// Pull side and owner side of a step: version lookup for the query, applying pushed rows, deciding which
// queried rows are outdated, packing the rows to return, refreshing cached rows and the final gather of
// every key's row into the caller's output.
// Reference: csrc/core/generate_query.cu:91-106, csrc/core/handle_query.cu:7-116,
// csrc/core/writeback.cu:8-56.
#include "kernels.h"

namespace hctr {
namespace {

constexpr int kBlock = 256;
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int VEC> struct RowVec;
template <> struct RowVec<4> { typedef floatx4 T; };
template <> struct RowVec<1> { typedef float T; };

__global__ __launch_bounds__(kBlock) void lookup_version(TableView t, BatchView c, version_t *__restrict__ q_ver) {
  const uint32_t u = blockIdx.x * kBlock + threadIdx.x;
  if (u >= *c.d_U) return;
  const slot_t o = c.uoff[u];
  q_ver[u] = o != kNoSlot ? t.ver[o] : kInvalidVersion;
}

template <typename K>
__global__ __launch_bounds__(kBlock) void unique_ids(int id_bits, BatchView c, index_t *__restrict__ q_idx) {
  const uint32_t u = blockIdx.x * kBlock + threadIdx.x;
  if (u >= *c.d_U) return;
  q_idx[u] = (index_t)(((const K *)c.ukey)[u] & (K)(((uint64_t)1 << id_bits) - 1));
}

// one group of LPR lanes per received row
template <int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void apply_remote(TableView t, const index_t *__restrict__ rg_idx,
                                                       const version_t *__restrict__ rg_cnt,
                                                       const embed_t *__restrict__ rg_val, uint32_t lo, uint32_t hi,
                                                       uint32_t *__restrict__ err) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const uint32_t k = lo + blockIdx.x * kGroups + threadIdx.x / LPR;
  if (k >= hi) return;
  const uint32_t gl = threadIdx.x % LPR, W = t.width;
  const uint64_t id = (uint64_t)rg_idx[k];
  slot_t o = kNoSlot;
  if (id < t.id_max && t.root[id] == t.rank) o = t.slot[id];
  if (o == kNoSlot) {
    if (gl == 0) atomicOr(err, 2u);
    return;
  }
  if (gl == 0) t.ver[o] += rg_cnt[k];
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC) {
    V *e = (V *)(t.emb + (size_t)o * W + col);
    *e = *e + *(const V *)(rg_val + (size_t)k * W + col);
  }
}

__global__ __launch_bounds__(kBlock) void decide_outdated(TableView t, const index_t *__restrict__ rq_idx,
                                                          const version_t *__restrict__ rq_ver, uint32_t q,
                                                          uint32_t self_lo, uint32_t self_hi,
                                                          uint32_t *__restrict__ outdated, uint32_t *__restrict__ err) {
  const uint32_t k = blockIdx.x * kBlock + threadIdx.x;
  if (k >= q) return;
  const uint64_t id = (uint64_t)rq_idx[k];
  slot_t o = kNoSlot;
  if (id < t.id_max && t.root[id] == t.rank) o = t.slot[id];
  if (o == kNoSlot) {
    atomicOr(err, 4u);
    outdated[k] = 0;
    return;
  }
  const version_t local = rq_ver[k], global = t.ver[o];
  const bool from_self = k >= self_lo && k < self_hi;
  const bool out = local == kInvalidVersion || local + t.pull_bound < global;
  outdated[k] = (out && !from_self) ? 1u : 0u;
}

template <int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void pack_rows(TableView t, const index_t *__restrict__ rq_idx,
                                                    const uint32_t *__restrict__ outdated,
                                                    const uint32_t *__restrict__ out_pos, uint32_t q,
                                                    version_t *__restrict__ ret_ver, embed_t *__restrict__ ret_val) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const uint32_t k = blockIdx.x * kGroups + threadIdx.x / LPR;
  if (k >= q || !outdated[k]) return;
  const uint32_t gl = threadIdx.x % LPR, W = t.width;
  const slot_t o = t.slot[(uint64_t)rq_idx[k]];
  const uint32_t pos = out_pos[k];
  if (gl == 0) ret_ver[pos] = t.ver[o];
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC)
    *(V *)(ret_val + (size_t)pos * W + col) = *(const V *)(t.emb + (size_t)o * W + col);
}

// Counts of the step's remote unique keys: [0] cached and fresh enough, [1] not stored here, [2] cached and
// refreshed.  Atomics on one address are served one after the other, so every thread counts its strided share in
// registers and a block adds its three totals once.
constexpr int kCountBlocks = 128;
__global__ __launch_bounds__(kBlock) void count_remote(TableView t, BatchView c, const uint32_t *__restrict__ got,
                                                       uint32_t *__restrict__ stats) {
  __shared__ uint32_t tot[3];
  if (threadIdx.x < 3) tot[threadIdx.x] = 0;
  __syncthreads();
  const uint32_t U = *c.d_U;
  uint32_t n0 = 0, n1 = 0, n2 = 0;
  for (uint32_t u = blockIdx.x * kBlock + threadIdx.x; u < U; u += kCountBlocks * kBlock) {
    const slot_t o = c.uoff[u];
    if (o == kNoSlot) n1++;
    else if ((uint32_t)o < t.n_cached) {
      if (got[u]) n2++;
      else n0++;
    }
  }
  for (int d = 32; d; d >>= 1) {
    n0 += __shfl_down(n0, d);
    n1 += __shfl_down(n1, d);
    n2 += __shfl_down(n2, d);
  }
  if (threadIdx.x % 64 == 0) {
    atomicAdd(&tot[0], n0);
    atomicAdd(&tot[1], n1);
    atomicAdd(&tot[2], n2);
  }
  __syncthreads();
  if (threadIdx.x < 3 && tot[threadIdx.x]) atomicAdd(&stats[threadIdx.x], tot[threadIdx.x]);
}

// one group per unique rank of the current batch
template <int VEC, int LPR>
__global__ __launch_bounds__(kBlock) void refresh(TableView t, BatchView c, PullArgs a, uint32_t *__restrict__ stats) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
  const uint32_t u = blockIdx.x * kGroups + threadIdx.x / LPR;
  if (u >= *c.d_U) return;
  const uint32_t gl = threadIdx.x % LPR, W = t.width;
  const slot_t o = c.uoff[u];
  const bool got = a.got[u] != 0;
  if (!got || o == kNoSlot) return;
  if ((uint32_t)o >= t.n_cached) { // an owned row can never come back as outdated
    if (gl == 0) atomicOr(&stats[3], 8u);
    return;
  }
  const uint32_t k = a.ret_i[u];
  if (gl == 0) t.ver[o] = a.in_ver[k];
  for (uint32_t col = gl * VEC; col < W; col += LPR * VEC)
    *(V *)(t.emb + (size_t)o * W + col) =
        *(const V *)(a.in_val + (size_t)k * W + col) + *(const V *)(t.pend + (size_t)o * W + col);
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
    const slot_t o = c.uoff[u];
    if (kLocalOnly || o != kNoSlot) src[k] = t.emb + (size_t)o * W;
    else src[k] = a.in_val + (size_t)a.ret_i[u] * W;
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

// Sum-pooled lookups: one group per bag of `bag` consecutive batch positions.  The rows of the bag are requested
// kPoolAhead at a time and added in position order (fp32, starting from the first row), so a bag costs one output
// row instead of `bag`.  Works in batch order, through the inverse index of the batch.
constexpr int kPoolAhead = 8;
template <int VEC, int LPR, bool kLocalOnly>
__global__ __launch_bounds__(kBlock) void gather_pooled(TableView t, BatchView c, PullArgs a, uint32_t bag,
                                                        uint32_t n_bags) {
  typedef typename RowVec<VEC>::T V;
  constexpr int kGroups = kBlock / LPR;
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
        const slot_t o = c.uoff[u];
        if (kLocalOnly || o != kNoSlot) src[k] = t.emb + (size_t)o * W;
        else src[k] = a.in_val + (size_t)a.ret_i[u] * W;
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

__global__ __launch_bounds__(kBlock) void copy_segments(const CopyDesc *__restrict__ d) {
  const CopyDesc cd = d[blockIdx.y];
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if ((((uintptr_t)cd.src | (uintptr_t)cd.dst | cd.bytes) & 15) == 0) {
    const uint4 *s = (const uint4 *)cd.src;
    uint4 *o = (uint4 *)cd.dst;
    for (size_t i = tid; i < cd.bytes / 16; i += stride) o[i] = s[i];
  } else {
    const uint32_t *s = (const uint32_t *)cd.src;
    uint32_t *o = (uint32_t *)cd.dst;
    for (size_t i = tid; i < cd.bytes / 4; i += stride) o[i] = s[i];
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

void launch_lookup_version(hipStream_t s, const TableView &t, const BatchView &cur, version_t *q_ver) {
  if (!cur.n) return;
  hipLaunchKernelGGL(lookup_version, dim3(div_up(cur.n, kBlock)), dim3(kBlock), 0, s, t, cur, q_ver);
  HCTR_HIP(hipGetLastError());
}

void launch_unique_ids(hipStream_t s, const KeyLayout &kl, const BatchView &cur, index_t *q_idx) {
  if (!cur.n) return;
  if (kl.wide) hipLaunchKernelGGL(unique_ids<uint64_t>, dim3(div_up(cur.n, kBlock)), dim3(kBlock), 0, s, kl.id_bits, cur, q_idx);
  else hipLaunchKernelGGL(unique_ids<uint32_t>, dim3(div_up(cur.n, kBlock)), dim3(kBlock), 0, s, kl.id_bits, cur, q_idx);
  HCTR_HIP(hipGetLastError());
}

void launch_apply_remote(hipStream_t s, const TableView &t, const index_t *rg_idx, const version_t *rg_cnt,
                         const embed_t *rg_val, uint32_t lo, uint32_t hi, uint32_t *err) {
  if (hi <= lo) return;
  const bool vec4 = t.width % 4 == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
#define CALL(V, L) \
  hipLaunchKernelGGL((apply_remote<V, L>), dim3(div_up(hi - lo, kBlock / L)), dim3(kBlock), 0, s, t, rg_idx, rg_cnt, rg_val, lo, hi, err)
  HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_decide_outdated(hipStream_t s, const TableView &t, const index_t *rq_idx, const version_t *rq_ver,
                            uint32_t q, uint32_t self_lo, uint32_t self_hi, uint32_t *outdated, uint32_t *err) {
  if (!q) return;
  hipLaunchKernelGGL(decide_outdated, dim3(div_up(q, kBlock)), dim3(kBlock), 0, s, t, rq_idx, rq_ver, q, self_lo,
                     self_hi, outdated, err);
  HCTR_HIP(hipGetLastError());
}

void launch_pack_rows(hipStream_t s, const TableView &t, const index_t *rq_idx, const uint32_t *outdated,
                      const uint32_t *out_pos, uint32_t q, version_t *ret_ver, embed_t *ret_val) {
  if (!q) return;
  const bool vec4 = t.width % 4 == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
#define CALL(V, L) \
  hipLaunchKernelGGL((pack_rows<V, L>), dim3(div_up(q, kBlock / L)), dim3(kBlock), 0, s, t, rq_idx, outdated, out_pos, q, ret_ver, ret_val)
  HCTR_DISPATCH_ROW(vec4, lpr, CALL);
#undef CALL
  HCTR_HIP(hipGetLastError());
}

void launch_refresh(hipStream_t s, const TableView &t, const BatchView &cur, uint32_t n_unique, const PullArgs &a,
                    uint32_t *stats) {
  if (!n_unique || !a.got) return;
  hipLaunchKernelGGL(count_remote, dim3(kCountBlocks), dim3(kBlock), 0, s, t, cur, a.got, stats);
  const bool vec4 = t.width % 4 == 0;
  const int lpr = lanes_for(t.width, vec4 ? 4 : 1);
#define CALL(V, L) \
  hipLaunchKernelGGL((refresh<V, L>), dim3(div_up(n_unique, kBlock / L)), dim3(kBlock), 0, s, t, cur, a, stats)
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

void launch_copies(hipStream_t s, const CopyDesc *descs_device, uint32_t n, size_t max_bytes) {
  if (!n || !max_bytes) return;
  const unsigned bx = (unsigned)std::min<size_t>(1024, (max_bytes / 16 + kBlock - 1) / kBlock + 1);
  hipLaunchKernelGGL(copy_segments, dim3(bx, n), dim3(kBlock), 0, s, descs_device);
  HCTR_HIP(hipGetLastError());
}

} // namespace hctr
