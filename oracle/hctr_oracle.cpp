// CPU restatement of HetuCTR's per-GPU embedding hot path.  TEST INFRASTRUCTURE ONLY.
//
// This file is the parity checker and the timed CPU baseline.  Nothing in the
// product (the HIP library, its C ABI, the hetuCTR python module) links, loads
// or calls it; only the test-suite, the smoke entry and the cpu_baseline leg of
// the benchmark do.
//
// It restates, for R logical ranks that live in one process and step in
// lock-step, what the reference does on R GPUs with NCCL in between.  Every
// exchange is a copy in source-rank order (csrc/core/all2all.cu:18-130).
// Citations are relative to the reference tree.
//
// Pinning status of each function (what checks it, beyond re-typing it):
//   init_values Zero/Uniform     closed form s*48271^(n+1) mod (2^31-1) in python
//                                ints and rationals (also committed as known answers)
//   init_values Normal/Truncated formula pinned by the inverse normal CDF of python's
//                                statistics.NormalDist in float64 (constants, sign,
//                                mirror and redraw rule); the bit pattern of CUDA's
//                                erfcinvf is not reproducible here: PARITY UNPINNED
//                                at bit level
//                                (oracle/_ref/libref_initializer.so, the reference's
//                                initializer.cu compiled against the image's rocThrust,
//                                is a cross-check only: rocThrust stands in for the
//                                CUDA Thrust the reference uses, so it pins nothing)
//   preprocess_index             numpy lexsort / unique / searchsorted, brute force
//   preprocess_gradient, generate_gradient, handle_*, write_back
//                                closed forms of tests/test_update.py (exact counts,
//                                1e-4 sums) with caches present, tests/check.py
//                                invariant, hand-computed staleness scenarios.
//                                Bounded staleness (bounds != 0) is exercised by no
//                                reference test with a value oracle: PARITY UNPINNED
//                                by the reference, pinned by hand scenarios only.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <numeric>
#include <string>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

typedef float embed_t;       // csrc/core/types.h:12
typedef long long version_t; // csrc/core/types.h:16
typedef long long index_t;   // csrc/core/types.h:19
typedef unsigned char worker_t; // csrc/core/types.h:28
const index_t kInvalidIndex = -1;                                              // types.h:22
const version_t kInvalidVersion = std::numeric_limits<version_t>::min();      // types.h:25

// ---------------------------------------------------------------------------------------------
// Table value initialisers (csrc/utils/initializer.cu:11-103).
// thrust::default_random_engine is minstd_rand: x <- 48271*x mod (2^31-1); seed 0 becomes state 1
// because the increment is 0.  discard(n) then one draw gives x_{n+1} = s*48271^(n+1) mod m.
// ---------------------------------------------------------------------------------------------
const uint64_t kLcgA = 48271ULL, kLcgM = 2147483647ULL;

inline uint64_t lcg_pow(uint64_t e) {
  uint64_t r = 1, b = kLcgA;
  while (e) {
    if (e & 1) r = r * b % kLcgM;
    b = b * b % kLcgM;
    e >>= 1;
  }
  return r;
}
inline uint32_t lcg_seed_state(unsigned int seed) {
  uint64_t s = seed % kLcgM;
  return s == 0 ? 1u : (uint32_t)s;
}
// state after `steps` advances from state x
inline uint32_t lcg_skip(uint32_t x, uint64_t steps) { return (uint32_t)(lcg_pow(steps) * x % kLcgM); }

// uniform_real_distribution<float>(a,b): (x-min)/(1+(max-min))*(b-a)+a, min=1, max=m-1.
// The multiply-add is written as one fused operation, which is what a GPU compiler emits for it.
inline float draw_uniform(uint32_t x, float a, float b) {
  float r = (float)(x - 1u);
  r /= (1.0f + (float)(uint32_t)(kLcgM - 2));
  return fmaf(r, b - a, a);
}

// inverse complementary error function, double precision: initial rational guess refined by
// Halley steps on erfc until converged.
double erfcinv_d(double y) {
  if (y <= 0) return INFINITY;
  if (y >= 2) return -INFINITY;
  double q = y < 1 ? y : 2 - y; // solve for q in (0,1], flip sign afterwards
  double t = std::sqrt(-2.0 * std::log(q / 2.0));
  double x = (t - (2.515517 + t * (0.802853 + t * 0.010328)) /
                      (1.0 + t * (1.432788 + t * (0.189269 + t * 0.001308)))) *
             0.70710678118654752440;
  for (int it = 0; it < 4; it++) {
    double err = std::erfc(x) - q;
    double d = -1.1283791670955126 * std::exp(-x * x);
    x -= err / (d - x * err); // Halley: f''/f' = -2x
  }
  return y < 1 ? x : -x;
}

// the direct-sampling normal used by device compilers: mean + sigma*(-+sqrt2)*erfcinv(2p)
inline float draw_normal(uint32_t x, float mean, float stddev) {
  const uint32_t range = (uint32_t)(kLcgM - 2);
  const float S1 = (float)(1.0 / (double)range);
  const float S2 = S1 / 2;
  float S3 = -1.4142135623730950488f;
  uint32_t u = x - 1u;
  if (u > range / 2) {
    u = range - u;
    S3 = -S3;
  }
  float p = fmaf((float)u, S1, S2);
  float e = (float)erfcinv_d((double)(2 * p));
  return fmaf(stddev * S3, e, mean);
}

void init_values(embed_t *out, size_t len, int type, float a, float b, unsigned int seed) {
  const uint32_t s0 = lcg_seed_state(seed);
#pragma omp parallel for schedule(static)
  for (long long n = 0; n < (long long)len; n++) {
    if (type == 0) { out[n] = 0.f; continue; }
    uint32_t x = lcg_skip(s0, (uint64_t)n + 1);
    if (type == 2) out[n] = draw_uniform(x, a, b);          // initializer.cu:11-27
    else if (type == 1) out[n] = draw_normal(x, a, b);      // initializer.cu:29-46
    else {                                                  // initializer.cu:48-70
      float r;
      for (;;) {
        r = draw_normal(x, a, b);
        // rng.seed(rng()): one more draw becomes the new state (never 0 for this engine)
        x = lcg_skip(x, 1);
        x = lcg_seed_state(x);
        if (!(r > a + 2 * b || r < a - 2 * b)) break;
        x = lcg_skip(x, 1);
      }
      out[n] = r;
    }
  }
}

// A zero-filled array whose pages the system hands out when they are first touched (calloc): a table of tens of
// millions of rows that starts from zeros costs memory and time only for the rows the test's batches reach.
template <typename T> struct ZeroArray {
  T *p = nullptr;
  size_t n = 0;
  ZeroArray() {}
  ZeroArray(const ZeroArray &) = delete;
  ZeroArray &operator=(const ZeroArray &) = delete;
  ZeroArray(ZeroArray &&o) noexcept : p(o.p), n(o.n) { o.p = nullptr; o.n = 0; }
  ~ZeroArray() { free(p); }
  void reset(size_t count) {
    free(p);
    p = (T *)calloc(count ? count : 1, sizeof(T));
    n = p ? count : 0;
  }
  T *data() { return p; }
  const T *data() const { return p; }
  size_t size() const { return n; }
  T &operator[](size_t i) { return p[i]; }
  const T &operator[](size_t i) const { return p[i]; }
  T *begin() { return p; }
};

// ---------------------------------------------------------------------------------------------
// Per-batch record (csrc/core/preprocess_struct.h:7-24)
// ---------------------------------------------------------------------------------------------
struct Batch {
  size_t N = 0, U = 0;
  std::vector<index_t> idx, unique, sorted_arg, run_start, idx_map, offset;
  std::vector<worker_t> root;
  std::vector<uint64_t> send_cnt, recv_cnt;         // query counts per owner / per requester
  std::vector<uint64_t> push_cnt, pushrecv_cnt;     // pushed rows per owner / per source
};

struct Rank {
  int rank = 0;
  size_t S = 0, C = 0; // stored rows, cached rows (offsets < C are cached)
  std::vector<index_t> store_ids;   // id at each offset
  std::vector<index_t> slot;        // id -> offset or -1 (stands for the hash map find)
  ZeroArray<embed_t> emb, pend;
  std::vector<version_t> ver, upd;
  Batch cur, prev;
  std::vector<index_t> need, prefix; // push plan of prev
  // send side
  std::vector<index_t> q_idx; std::vector<version_t> q_ver;
  std::vector<index_t> g_idx; std::vector<version_t> g_cnt; std::vector<embed_t> g_val;
  // receive side
  std::vector<index_t> rq_idx; std::vector<version_t> rq_ver; std::vector<uint64_t> rq_seg; // R+1
  std::vector<index_t> rg_idx; std::vector<version_t> rg_cnt; std::vector<embed_t> rg_val; std::vector<uint64_t> rg_seg;
  std::vector<index_t> outdated;                 // per received query
  std::vector<version_t> ret_ver; std::vector<embed_t> ret_val; std::vector<uint64_t> ret_seg; // rows I return, per requester
  // requester side of the return
  std::vector<index_t> got;                      // per unique of cur
  std::vector<index_t> ret_i;
  std::vector<version_t> in_ver; std::vector<embed_t> in_val;
  // counters of the last step
  long long st_hit = 0, st_miss = 0, st_refresh = 0, st_pushed = 0, st_served = 0, st_grad_recv = 0;
};

struct Group {
  int R = 1;
  size_t IDMax = 0, W = 0;
  version_t pull_bound = 0, push_bound = 0;
  embed_t lr = 0;
  std::vector<worker_t> root;
  std::vector<Rank> ranks;
  bool parallel = false; // OpenMP inside the heavy loops (timed baseline); results identical
  std::string err;
};

// ---- csrc/core/table_initialize.cu:66-114 -----------------------------------------------------
bool init_rank(Group &g, Rank &rk, const index_t *storage, size_t S, int init_type, float a, float b,
               unsigned seed) {
  rk.S = S;
  rk.store_ids.resize(S);
  // stable partition: ids whose owner is another rank first, order kept (:81)
  size_t c = 0;
  for (size_t i = 0; i < S; i++) {
    if (storage[i] < 0 || (size_t)storage[i] >= g.IDMax) { g.err = "storage id out of range"; return false; }
    if (g.root[storage[i]] != rk.rank) rk.store_ids[c++] = storage[i];
  }
  rk.C = c;
  for (size_t i = 0; i < S; i++)
    if (g.root[storage[i]] == rk.rank) rk.store_ids[c++] = storage[i];
  rk.slot.assign(g.IDMax, kInvalidIndex);
  for (size_t o = 0; o < S; o++) rk.slot[rk.store_ids[o]] = (index_t)o; // insert (key[i] -> i) (:84-87)
  rk.emb.reset(S * g.W);
  rk.pend.reset(rk.C * g.W);                                             // :102-103
  if (rk.emb.size() != S * g.W || rk.pend.size() != rk.C * g.W) { g.err = "out of memory"; return false; }
  rk.upd.assign(rk.C, 0);                                                // :104-105
  rk.ver.resize(S);
  for (size_t o = 0; o < S; o++) rk.ver[o] = o < rk.C ? kInvalidVersion : 0; // :108-112
  if (init_type != 0) init_values(rk.emb.data(), S * g.W, init_type, a, b, seed); // :156, value depends on offset
  return true;
}

// ---- csrc/core/preprocess.cu:92-141 -----------------------------------------------------------
void preprocess_index(Group &g, Rank &rk, const index_t *keys, size_t N) {
  Batch &c = rk.cur;
  const int R = g.R;
  c.N = N;
  c.idx.assign(keys, keys + N);
  // sort key id + IDMax*root[id] (:17); stable, so equal keys stay in ascending position (:105-109)
  std::vector<uint64_t> skey(N);
  for (size_t i = 0; i < N; i++) skey[i] = (uint64_t)keys[i] + (uint64_t)g.IDMax * g.root[keys[i]];
  c.sorted_arg.resize(N);
  std::iota(c.sorted_arg.begin(), c.sorted_arg.end(), 0);
  if (g.parallel && N > (1u << 16)) {
    // LSD radix sort, 8-bit digits: stable by construction, same result as stable_sort
    uint64_t maxk = (uint64_t)g.IDMax * (uint64_t)R;
    int bits = 1; while (bits < 64 && (maxk >> bits)) bits++;
    std::vector<uint64_t> k2(N); std::vector<index_t> a2(N);
    int nt = 1;
#ifdef _OPENMP
    nt = omp_get_max_threads();
#endif
    std::vector<size_t> hist((size_t)nt * 256);
    for (int sh = 0; sh < bits; sh += 8) {
      std::fill(hist.begin(), hist.end(), 0);
#pragma omp parallel num_threads(nt)
      {
        int t = 0;
#ifdef _OPENMP
        t = omp_get_thread_num();
#endif
        size_t lo = N * t / nt, hi = N * (t + 1) / nt;
        size_t *h = &hist[(size_t)t * 256];
        for (size_t i = lo; i < hi; i++) h[(skey[i] >> sh) & 255]++;
#pragma omp barrier
#pragma omp single
        {
          size_t acc = 0;
          for (int d = 0; d < 256; d++)
            for (int tt = 0; tt < nt; tt++) { size_t v = hist[(size_t)tt * 256 + d]; hist[(size_t)tt * 256 + d] = acc; acc += v; }
        }
        for (size_t i = lo; i < hi; i++) {
          size_t p = h[(skey[i] >> sh) & 255]++;
          k2[p] = skey[i]; a2[p] = c.sorted_arg[i];
        }
      }
      skey.swap(k2); c.sorted_arg.swap(a2);
    }
  } else {
    std::stable_sort(c.sorted_arg.begin(), c.sorted_arg.end(),
                     [&](index_t x, index_t y) { return skey[x] < skey[y]; });
    std::vector<uint64_t> k2(N);
    for (size_t j = 0; j < N; j++) k2[j] = skey[c.sorted_arg[j]];
    skey.swap(k2);
  }
  // run-length encode the sorted ids (:115-117), exclusive scan of the lengths (:124-125)
  c.unique.clear(); c.run_start.clear();
  for (size_t j = 0; j < N; j++)
    if (j == 0 || skey[j] != skey[j - 1]) { c.unique.push_back(keys[c.sorted_arg[j]]); c.run_start.push_back((index_t)j); }
  c.U = c.unique.size();
  c.run_start.push_back((index_t)N);
  // per unique: owner and resident offset (:49-57); bucket starts at owner boundaries (:58-67)
  c.root.resize(c.U); c.offset.resize(c.U);
  std::vector<uint64_t> lo(R + 1, c.U);
  int r_prev = -1;
  for (size_t u = 0; u < c.U; u++) {
    int r = g.root[c.unique[u]];
    c.root[u] = (worker_t)r;
    c.offset[u] = rk.slot[c.unique[u]];
    for (int i = r_prev + 1; i <= r; i++) lo[i] = u;
    r_prev = r;
  }
  if (c.U == 0) std::fill(lo.begin(), lo.end(), 0); // :93-95
  // inverse index: lower bound inside the owner's segment (:71-90)
  c.idx_map.resize(N);
#pragma omp parallel for schedule(static) if (g.parallel)
  for (long long i = 0; i < (long long)N; i++) {
    int r = g.root[keys[i]];
    const index_t *b = c.unique.data();
    c.idx_map[i] = std::lower_bound(b + lo[r], b + lo[r + 1], keys[i]) - b;
  }
  // offsets -> sizes (:22-32)
  c.send_cnt.assign(R + 1, 0);
  for (int i = 0; i < R; i++) c.send_cnt[i] = lo[i + 1] - lo[i];
}

// ---- csrc/core/preprocess.cu:148-182 ----------------------------------------------------------
void preprocess_gradient(Group &g, Rank &rk) {
  Batch &p = rk.prev;
  rk.need.assign(p.U, 0); rk.prefix.assign(p.U, 0);
  p.push_cnt.assign(g.R + 1, 0);
  for (size_t u = 0; u < p.U; u++) {
    version_t cnt = p.run_start[u + 1] - p.run_start[u];
    index_t o = p.offset[u];
    index_t need;
    if (p.root[u] == rk.rank) need = 0;
    else if (o == kInvalidIndex) need = 1;
    else need = (rk.upd[o] + cnt <= g.push_bound) ? 0 : 1;
    rk.need[u] = need;
    if (need) p.push_cnt[p.root[u]]++;
  }
  index_t acc = 0;
  for (size_t u = 0; u < p.U; u++) { rk.prefix[u] = acc; acc += rk.need[u]; }
}

// ---- csrc/core/generate_query.cu:8-89 ---------------------------------------------------------
void generate_gradient(Group &g, Rank &rk, const embed_t *grad) {
  Batch &p = rk.prev;
  const size_t W = g.W;
  size_t npush = 0;
  for (int i = 0; i < g.R; i++) npush += p.push_cnt.empty() ? 0 : p.push_cnt[i];
  rk.g_idx.assign(npush, 0); rk.g_cnt.assign(npush, 0); rk.g_val.assign(npush * W, 0.f);
  rk.st_pushed = (long long)npush;
  const embed_t neg_lr = -g.lr;
#pragma omp parallel for schedule(dynamic, 256) if (g.parallel)
  for (long long uu = 0; uu < (long long)p.U; uu++) {
    size_t u = (size_t)uu;
    index_t o = p.offset[u];
    bool need = rk.need[u] != 0;
    int type = o == kInvalidIndex ? 0 : ((size_t)o >= rk.C ? 1 : (need ? 2 : 3)); // :18-25
    version_t cnt = p.run_start[u + 1] - p.run_start[u];
    // counters (:51-83)
    if (type == 1) rk.ver[o] += cnt;
    else if (type >= 2) {
      rk.upd[o] += cnt;
      if (type == 2) { cnt = rk.upd[o]; rk.upd[o] = 0; rk.ver[o] += cnt; }
    }
    index_t q = rk.prefix[u];
    if (need) { rk.g_idx[q] = p.unique[u]; rk.g_cnt[q] = cnt; }
    // values (:33-48): serial sum in run order, one multiply by -lr, one add
    for (size_t w = 0; w < W; w++) {
      embed_t sum = 0;
      for (index_t j = p.run_start[u]; j < p.run_start[u + 1]; j++) sum += grad[(size_t)p.sorted_arg[j] * W + w];
      sum *= neg_lr;
      if (type != 0) rk.emb[(size_t)o * W + w] += sum;
      else rk.g_val[(size_t)q * W + w] = sum;
      if (type >= 2) rk.pend[(size_t)o * W + w] += sum;
      if (type == 2) { rk.g_val[(size_t)q * W + w] = rk.pend[(size_t)o * W + w]; rk.pend[(size_t)o * W + w] = 0; }
    }
  }
}

// ---- csrc/core/generate_query.cu:91-106 -------------------------------------------------------
void generate_query(Group &, Rank &rk) {
  Batch &c = rk.cur;
  rk.q_idx = c.unique;
  rk.q_ver.resize(c.U);
  for (size_t u = 0; u < c.U; u++) rk.q_ver[u] = c.offset[u] != kInvalidIndex ? rk.ver[c.offset[u]] : kInvalidVersion;
}

// ---- csrc/core/all2all.cu:18-87: receive buffers are the senders' buckets in source-rank order --
void exchange_query(Group &g) {
  const int R = g.R; const size_t W = g.W;
  for (int d = 0; d < R; d++) {
    Rank &dst = g.ranks[d];
    dst.rq_idx.clear(); dst.rq_ver.clear(); dst.rq_seg.assign(R + 1, 0);
    dst.rg_idx.clear(); dst.rg_cnt.clear(); dst.rg_val.clear(); dst.rg_seg.assign(R + 1, 0);
    for (int s = 0; s < R; s++) {
      Rank &src = g.ranks[s];
      size_t qlo = 0; for (int i = 0; i < d; i++) qlo += src.cur.send_cnt[i];
      size_t qn = src.cur.send_cnt[d];
      dst.rq_idx.insert(dst.rq_idx.end(), src.q_idx.begin() + qlo, src.q_idx.begin() + qlo + qn);
      dst.rq_ver.insert(dst.rq_ver.end(), src.q_ver.begin() + qlo, src.q_ver.begin() + qlo + qn);
      dst.rq_seg[s + 1] = dst.rq_idx.size();
      size_t glo = 0, gn = 0;
      if (!src.prev.push_cnt.empty()) { for (int i = 0; i < d; i++) glo += src.prev.push_cnt[i]; gn = src.prev.push_cnt[d]; }
      dst.rg_idx.insert(dst.rg_idx.end(), src.g_idx.begin() + glo, src.g_idx.begin() + glo + gn);
      dst.rg_cnt.insert(dst.rg_cnt.end(), src.g_cnt.begin() + glo, src.g_cnt.begin() + glo + gn);
      dst.rg_val.insert(dst.rg_val.end(), src.g_val.begin() + glo * W, src.g_val.begin() + (glo + gn) * W);
      dst.rg_seg[s + 1] = dst.rg_idx.size();
    }
  }
}

// ---- csrc/core/handle_query.cu:81-116: one source after the other, in rank order ---------------
bool handle_gradient(Group &g, Rank &rk) {
  const size_t W = g.W;
  rk.st_grad_recv = (long long)rk.rg_idx.size();
  for (size_t k = 0; k < rk.rg_idx.size(); k++) {
    index_t id = rk.rg_idx[k];
    index_t o = rk.slot[id];
    if (g.root[id] != rk.rank || o == kInvalidIndex) { g.err = "pushed row is not owned and stored by its destination"; return false; }
    rk.ver[o] += rk.rg_cnt[k];
    for (size_t w = 0; w < W; w++) rk.emb[(size_t)o * W + w] += rk.rg_val[k * W + w];
  }
  return true;
}

// ---- csrc/core/handle_query.cu:7-78 ------------------------------------------------------------
bool handle_query(Group &g, Rank &rk) {
  const size_t W = g.W; const int R = g.R;
  size_t Q = rk.rq_idx.size();
  rk.outdated.assign(Q, 0);
  rk.ret_ver.clear(); rk.ret_val.clear(); rk.ret_seg.assign(R + 1, 0);
  size_t self_lo = rk.rq_seg[rk.rank], self_hi = rk.rq_seg[rk.rank + 1];
  for (int s = 0; s < R; s++) {
    for (size_t k = rk.rq_seg[s]; k < rk.rq_seg[s + 1]; k++) {
      index_t id = rk.rq_idx[k];
      index_t o = rk.slot[id];
      if (g.root[id] != rk.rank || o == kInvalidIndex) { g.err = "queried row is not owned and stored by its destination"; return false; }
      version_t local = rk.rq_ver[k], global = rk.ver[o];
      bool from_self = k >= self_lo && k < self_hi;
      bool out = (local == kInvalidVersion || local + g.pull_bound < global) && !from_self; // :17-20
      rk.outdated[k] = out;
      if (out) {                                                                           // :24-40
        rk.ret_ver.push_back(global);
        rk.ret_val.insert(rk.ret_val.end(), rk.emb.begin() + (size_t)o * W, rk.emb.begin() + (size_t)(o + 1) * W);
      }
    }
    rk.ret_seg[s + 1] = rk.ret_ver.size();
  }
  rk.st_served = (long long)rk.ret_ver.size();
  return true;
}

// ---- csrc/core/all2all.cu:89-130 ---------------------------------------------------------------
void exchange_return(Group &g) {
  const int R = g.R; const size_t W = g.W;
  for (int s = 0; s < R; s++) { // s = requester
    Rank &req = g.ranks[s];
    req.got.clear(); req.in_ver.clear(); req.in_val.clear();
    for (int d = 0; d < R; d++) { // d = owner, in rank order
      Rank &own = g.ranks[d];
      req.got.insert(req.got.end(), own.outdated.begin() + own.rq_seg[s], own.outdated.begin() + own.rq_seg[s + 1]);
      req.in_ver.insert(req.in_ver.end(), own.ret_ver.begin() + own.ret_seg[s], own.ret_ver.begin() + own.ret_seg[s + 1]);
      req.in_val.insert(req.in_val.end(), own.ret_val.begin() + own.ret_seg[s] * W, own.ret_val.begin() + own.ret_seg[s + 1] * W);
    }
  }
}

// ---- csrc/core/writeback.cu:8-56 ---------------------------------------------------------------
bool write_back(Group &g, Rank &rk, embed_t *dst) {
  Batch &c = rk.cur; const size_t W = g.W;
  rk.ret_i.assign(c.U, 0);
  index_t acc = 0;
  rk.st_hit = rk.st_miss = rk.st_refresh = 0;
  for (size_t u = 0; u < c.U; u++) { rk.ret_i[u] = acc; acc += rk.got[u]; }
  for (size_t u = 0; u < c.U; u++) {
    if (c.root[u] != rk.rank) {
      if (c.offset[u] == kInvalidIndex) rk.st_miss++;
      else if (rk.got[u]) rk.st_refresh++;
      else rk.st_hit++;
    }
    if (!rk.got[u]) continue;
    index_t o = c.offset[u];
    if (o == kInvalidIndex) continue;
    if ((size_t)o >= rk.C) { g.err = "an owned row came back as outdated"; return false; }
    size_t k = (size_t)rk.ret_i[u];
    rk.ver[o] = rk.in_ver[k];
    for (size_t w = 0; w < W; w++) rk.emb[(size_t)o * W + w] = rk.in_val[k * W + w] + rk.pend[(size_t)o * W + w];
  }
  if (!dst) return true;
#pragma omp parallel for schedule(static) if (g.parallel)
  for (long long i = 0; i < (long long)c.N; i++) {
    size_t u = (size_t)c.idx_map[i];
    index_t o = c.offset[u];
    const embed_t *src = o == kInvalidIndex ? &rk.in_val[(size_t)rk.ret_i[u] * W] : &rk.emb[(size_t)o * W];
    memcpy(dst + (size_t)i * W, src, W * sizeof(embed_t));
  }
  return true;
}

thread_local std::string g_last_error;

} // namespace

extern "C" {

const char *orc_last_error() { return g_last_error.c_str(); }

void orc_init_values(float *out, size_t len, int type, float a, float b, unsigned int seed) {
  init_values(out, len, type, a, b, seed);
}

// storage: R pointers, n_storage: R sizes.  init_type: 0 Zero, 1 Normal, 2 Uniform, 3 TruncatedNormal
void *orc_create(int R, size_t length, size_t width, long long pull_bound, long long push_bound,
                 const unsigned char *root_arr, const long long *const *storage, const size_t *n_storage,
                 int init_type, float a, float b, float lr, unsigned int seed) {
  Group *g = new Group();
  g->R = R; g->IDMax = length; g->W = width; g->pull_bound = pull_bound; g->push_bound = push_bound; g->lr = lr;
  g->root.assign(root_arr, root_arr + length);
  for (size_t i = 0; i < length; i++)
    if (g->root[i] >= R) { g_last_error = "root_arr entry >= nrank"; delete g; return nullptr; }
  g->ranks.resize(R);
  for (int r = 0; r < R; r++) {
    g->ranks[r].rank = r;
    if (!init_rank(*g, g->ranks[r], storage[r], n_storage[r], init_type, a, b, seed)) { g_last_error = g->err; delete g; return nullptr; }
    for (Batch *bt : {&g->ranks[r].cur, &g->ranks[r].prev}) {
      bt->run_start.assign(1, 0); bt->send_cnt.assign(R + 1, 0); bt->recv_cnt.assign(R + 1, 0);
      bt->push_cnt.assign(R + 1, 0); bt->pushrecv_cnt.assign(R + 1, 0);
    }
  }
  // every id a rank owns must be resident on it (the reference asserts this only when serving)
  for (size_t i = 0; i < length; i++)
    if (g->ranks[g->root[i]].slot[i] == kInvalidIndex) { g_last_error = "an id is missing from its owner's storage_arr"; delete g; return nullptr; }
  return g;
}

void orc_destroy(void *h) { delete (Group *)h; }
void orc_set_parallel(void *h, int on) { ((Group *)h)->parallel = on != 0; }

// csrc/core/hetu_gpu_table.cu:43-65 for all ranks in lock-step
int orc_preprocess(void *h, const long long *const *keys, const size_t *n) {
  Group &g = *(Group *)h;
  for (int r = 0; r < g.R; r++)
    for (size_t i = 0; i < n[r]; i++)
      if (keys[r][i] < 0 || (size_t)keys[r][i] >= g.IDMax) { g_last_error = "key out of range"; return 1; }
  for (int r = 0; r < g.R; r++) {
    Rank &rk = g.ranks[r];
    std::swap(rk.cur, rk.prev);
    preprocess_index(g, rk, keys[r], n[r]);
  }
  for (int r = 0; r < g.R; r++) {
    g.ranks[r].cur.recv_cnt.assign(g.R + 1, 0);
    for (int s = 0; s < g.R; s++) g.ranks[r].cur.recv_cnt[s] = g.ranks[s].cur.send_cnt[r];
  }
  for (int r = 0; r < g.R; r++) preprocess_gradient(g, g.ranks[r]);
  for (int r = 0; r < g.R; r++) {
    g.ranks[r].prev.pushrecv_cnt.assign(g.R + 1, 0);
    for (int s = 0; s < g.R; s++) g.ranks[r].prev.pushrecv_cnt[s] = g.ranks[s].prev.push_cnt[r];
  }
  return 0;
}

// csrc/core/hetu_gpu_table.cu:9-41 for all ranks in lock-step.  grads[r] == NULL: inference on rank r.
int orc_push_pull(void *h, const float *const *grads, float *const *dsts) {
  Group &g = *(Group *)h;
  for (int r = 0; r < g.R; r++) {
    Rank &rk = g.ranks[r];
    if (!grads[r]) { // :14-21
      rk.prev.N = 0; rk.prev.U = 0;
      rk.prev.push_cnt.assign(g.R + 1, 0); rk.prev.pushrecv_cnt.assign(g.R + 1, 0);
    }
    generate_gradient(g, rk, grads[r]);
    generate_query(g, rk);
  }
  exchange_query(g);
  for (int r = 0; r < g.R; r++) if (!handle_gradient(g, g.ranks[r])) { g_last_error = g.err; return 1; }
  for (int r = 0; r < g.R; r++) if (!handle_query(g, g.ranks[r])) { g_last_error = g.err; return 1; }
  exchange_return(g);
  for (int r = 0; r < g.R; r++) if (!write_back(g, g.ranks[r], dsts[r])) { g_last_error = g.err; return 1; }
  return 0;
}

// Introspection.  Returns the element count; copies min(count, cap) elements.  Integer items are
// int64, item 16/17 are float.
//  0 unique  1 sorted_arg  2 run_start(U+1)  3 idx_map  4 root  5 offset  6 send_cnt(R)  7 recv_cnt(R)
//  8 need_update(prev)  9 update_prefix(prev)  10 push_cnt(R)  11 pushrecv_cnt(R)
// 12 outdated flags of received queries  13 got flags per unique  14 version(S)  15 updates(C)
// 16 embedding(S*W)  17 pending(C*W)  18 ids in offset order(S)  19 stats{hit,miss,refresh,pushed,served,grad_recv}
// 20 sizes {N,U,Nprev,Uprev,S,C}  21 keys of the batch
long long orc_fetch(void *h, int rank, int which, void *out, size_t cap) {
  Group &g = *(Group *)h; Rank &rk = g.ranks[rank];
  auto put64 = [&](const auto &v, size_t n) -> long long {
    long long *o = (long long *)out;
    for (size_t i = 0; i < n && i < cap; i++) o[i] = (long long)v[i];
    return (long long)n;
  };
  auto putf = [&](const ZeroArray<embed_t> &v) -> long long {
    memcpy(out, v.data(), std::min(cap, v.size()) * sizeof(embed_t));
    return (long long)v.size();
  };
  switch (which) {
    case 0: return put64(rk.cur.unique, rk.cur.U);
    case 1: return put64(rk.cur.sorted_arg, rk.cur.N);
    case 2: return put64(rk.cur.run_start, rk.cur.U + 1);
    case 3: return put64(rk.cur.idx_map, rk.cur.N);
    case 4: return put64(rk.cur.root, rk.cur.U);
    case 5: return put64(rk.cur.offset, rk.cur.U);
    case 6: return put64(rk.cur.send_cnt, (size_t)g.R);
    case 7: return put64(rk.cur.recv_cnt, (size_t)g.R);
    case 8: return put64(rk.need, rk.need.size());
    case 9: return put64(rk.prefix, rk.prefix.size());
    case 10: return put64(rk.prev.push_cnt, (size_t)g.R);
    case 11: return put64(rk.prev.pushrecv_cnt, (size_t)g.R);
    case 12: return put64(rk.outdated, rk.outdated.size());
    case 13: return put64(rk.got, rk.got.size());
    case 14: return put64(rk.ver, rk.S);
    case 15: return put64(rk.upd, rk.C);
    case 16: return putf(rk.emb);
    case 17: return putf(rk.pend);
    case 18: return put64(rk.store_ids, rk.S);
    case 19: { long long s[6] = {rk.st_hit, rk.st_miss, rk.st_refresh, rk.st_pushed, rk.st_served, rk.st_grad_recv}; return put64(s, 6); }
    case 20: { long long s[6] = {(long long)rk.cur.N, (long long)rk.cur.U, (long long)rk.prev.N, (long long)rk.prev.U, (long long)rk.S, (long long)rk.C}; return put64(s, 6); }
    case 21: return put64(rk.cur.idx, rk.cur.N);
  }
  return -1;
}

int orc_num_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

} // extern "C"
