// Offline partitioner (see partition.h).  The two sweeps are recurrences: every decision reads the part sizes and
// counters that all earlier moves of the same sweep changed, and every score is a chain of float operations that
// starts from those sizes, so the order of visits and of operations is the result.  They run on the host, one
// sample / embedding after the other, over a layout that makes a visit cheap.  What has no such order (the priority
// of every (part, embedding) pair and the sorted cache candidates per part) runs on the GPU.
#include "partition.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>

#include "radix_sort.h"

namespace hctr {
namespace {

// The C library's rand() (glibc, default 128-byte state): 31 words, x[f] += x[r] with the two cursors 3 apart,
// result = the new word >> 1; seeded by x[i] = 16807 * x[i-1] mod (2^31 - 1) and 310 discarded results.  The
// reference draws the initial assignment from rand() without seeding it (partition.cc:70,77), which is srand(1).
class LibcRand {
public:
  explicit LibcRand(unsigned seed) {
    int64_t w = (int32_t)(seed ? seed : 1u);
    st_[0] = (uint32_t)w;
    for (int i = 1; i < 31; i++) {
      w = (16807 * w) % 2147483647;
      if (w < 0) w += 2147483647;
      st_[i] = (uint32_t)w;
    }
    f_ = 3;
    r_ = 0;
    for (int i = 0; i < 310; i++) next();
  }
  int next() {
    const uint32_t v = (st_[f_] += st_[r_]);
    f_ = f_ == 30 ? 0 : f_ + 1;
    r_ = r_ == 30 ? 0 : r_ + 1;
    return (int)(v >> 1);
  }

private:
  uint32_t st_[31];
  int f_, r_;
};

// host threads a parallel step gets when it asks for `want`: at most 16 and at most what the machine has
size_t thread_count(size_t want) {
  const size_t hw = std::thread::hardware_concurrency();
  return std::max<size_t>(1, std::min<size_t>({want, hw ? hw : 1, 16}));
}

// runs fn(t, nthreads) on thread_count(want) host threads
template <typename F> void on_threads(size_t want, F &&fn) {
  const size_t nt = thread_count(want);
  std::vector<std::thread> pool;
  for (size_t t = 1; t < nt; t++) pool.emplace_back([&fn, t, nt] { fn(t, nt); });
  fn(0, nt);
  for (auto &th : pool) th.join();
}

int first_largest(const float *v, int n) { // partition.cc:17-24
  int r = 0;
  for (int i = 1; i < n; i++)
    if (v[i] > v[r]) r = i;
  return r;
}

} // namespace

Partitioner::Partitioner(const int32_t *d, size_t nd, size_t ns, const float *comm_mat, int np, int bs, unsigned seed)
    : n_part(np), batch(bs), n_data(nd), n_slot(ns) {
  HCTR_CHECK(d && comm_mat, "partition: null argument");
  HCTR_CHECK(np >= 1 && np <= 256, "partition: n_part must be in 1..256");
  HCTR_CHECK(bs >= 1, "partition: batch_size must be positive");
  HCTR_CHECK(ns >= 1 && nd >= (size_t)np, "partition: needs at least n_part samples and one slot");
  HCTR_CHECK(nd * ns < (1ull << 31), "partition: samples x slots must stay below 2^31");
  const size_t n_edge = nd * ns;
  int32_t top = 0, low = 0;
  for (size_t i = 0; i < n_edge; i++) {
    top = std::max(top, d[i]);
    low = std::min(low, d[i]);
  }
  HCTR_CHECK(low >= 0, "partition: negative embedding id");
  n_embed = (size_t)top + 1; // partition.cc:33-37
  HCTR_CHECK(n_embed >= (size_t)np, "partition: fewer embeddings than parts");
  for (int i = 0; i < np * np; i++) HCTR_CHECK(std::isfinite(comm_mat[i]), "partition: comm_mat must be finite");
  data.assign(d, d + n_edge);
  comm.assign(comm_mat, comm_mat + (size_t)np * np);
  comm_t.resize(comm.size());
  for (int i = 0; i < np; i++)
    for (int j = 0; j < np; j++) comm_t[(size_t)j * np + i] = comm[(size_t)i * np + j];

  // partition.cc:59-65: soft[i] = (1 - (1 - i/m)^batch) * m / batch below m = n_data / n_part, 1 from there on;
  // the power by repeated squaring in float (partition.cc:7-15)
  const size_t m = nd / np;
  soft.assign(nd, 1.0f);
  for (size_t i = 0; i < m; i++) {
    float sq = (float)(1.0 - (double)((float)i / (float)m)), pw = 1.0f;
    for (int e = bs; e; e >>= 1) {
      if (e & 1) pw *= sq;
      sq *= sq;
    }
    float v = 1 - pw;
    v *= (float)m / (float)bs;
    soft[i] = v;
  }
  dsoft.assign(nd + 1, 0.0f);
  for (size_t i = 0; i < nd; i++) dsoft[i] = soft_at((int64_t)i + 1) - soft[i];

  // partition.cc:66-80: samples first, then embeddings, one rand() each
  LibcRand rnd(seed);
  res_data.resize(nd);
  res_embed.resize(n_embed);
  cnt_data.assign(np, 0);
  cnt_embed.assign(np, 0);
  // the table is zeroed by several threads: first touch of a gigabyte from one thread is the slowest step otherwise
  cnt.resize(n_embed * (size_t)np);
  on_threads(16, [&](size_t t, size_t nt) {
    const size_t lo = cnt.size() * t / nt, hi = cnt.size() * (t + 1) / nt;
    memset(cnt.data() + lo, 0, (hi - lo) * sizeof(int32_t));
  });
  for (size_t i = 0; i < nd; i++) res_data[i] = rnd.next() % np;
  constexpr size_t kAhead = 8; // samples whose counter rows are requested before they are counted
  for (size_t i = 0; i < nd; i++) {
    if (i + kAhead < nd)
      for (size_t s = 0; s < ns; s++) __builtin_prefetch(&cnt[(size_t)d[(i + kAhead) * ns + s] * np], 1);
    const int p = res_data[i];
    cnt_data[p]++;
    for (size_t s = 0; s < ns; s++) cnt[(size_t)d[i * ns + s] * np + p]++;
  }
  for (size_t i = 0; i < n_embed; i++) {
    const int p = rnd.next() % np;
    res_embed[i] = p;
    cnt_embed[p]++;
  }
  // partition.cc:82-83: integer quotient, double division, kept as float
  alpha = (float)(-100.0 / (double)(nd / np));
  beta = (float)(-100.0 / (double)(n_embed / np));
}

template <int PC> void Partitioner::refine_data_sweep() {
  const int P = PC ? PC : n_part;
  const size_t S = n_slot;
  std::vector<float> score_v(P);
  float *score = score_v.data();
  constexpr size_t kAhead = 6; // samples whose counter rows are requested before they are needed
  for (size_t i = 0; i < n_data; i++) {
    if (i + kAhead < n_data) {
      const int32_t *nx = &data[(i + kAhead) * S];
      for (size_t s = 0; s < S; s++) {
        __builtin_prefetch(&cnt[(size_t)nx[s] * P], 1);
        __builtin_prefetch(&res_embed[nx[s]], 0);
      }
    }
    const int32_t *row = &data[i * S];
    const int old = res_data[i];
    for (int k = 0; k < P; k++) score[k] = alpha * (float)(cnt_data[k] - (k == old));
    for (size_t s = 0; s < S; s++) {
      const int32_t *c = &cnt[(size_t)row[s] * P];
      const float *cm = &comm_t[(size_t)res_embed[row[s]] * P]; // cm[k] = comm[k][owner of the embedding]
      for (int k = 0; k < P; k++) {
        // what one more sample of part k using this embedding adds to the part's soft count, not counting this sample
        const int64_t use = (int64_t)c[k] - (k == old);
        const float step = use < (int64_t)n_data ? dsoft[use] : 0.0f;
        score[k] -= step * cm[k];
      }
    }
    const int to = first_largest(score, P);
    if (to != old) {
      cnt_data[old]--;
      cnt_data[to]++;
      for (size_t s = 0; s < S; s++) {
        int32_t *c = &cnt[(size_t)row[s] * P];
        c[to]++;
        c[old]--;
      }
      res_data[i] = to;
    }
  }
}

void Partitioner::refine_data() {
  switch (n_part) {
  case 2: refine_data_sweep<2>(); break;
  case 4: refine_data_sweep<4>(); break;
  case 8: refine_data_sweep<8>(); break;
  case 16: refine_data_sweep<16>(); break;
  default: refine_data_sweep<0>();
  }
}

// partition.cc:123-131.  The sum for owner part p runs over (viewing part i != p, embedding j owned by p) in that
// nesting order.  Unused (part, embedding) pairs add soft[0] = 0 and are left out.  The counter table is read once,
// by threads over ranges of j that keep the nonzero terms per (p, i); a chain then adds its terms range after range.
std::vector<float> Partitioner::embed_weight_now() const {
  const int P = n_part;
  const size_t nt_used = thread_count(16);
  std::vector<std::vector<std::vector<float>>> terms(nt_used, std::vector<std::vector<float>>((size_t)P * P)); // [thread][p * P + i]
  on_threads(nt_used, [&](size_t t, size_t nt) {
    auto &mine = terms[t];
    const size_t lo = n_embed * t / nt, hi = n_embed * (t + 1) / nt;
    for (size_t j = lo; j < hi; j++) {
      const int32_t *c = &cnt[j * P];
      const int p = res_embed[j];
      for (int i = 0; i < P; i++)
        if (c[i] != 0 && i != p) mine[(size_t)p * P + i].push_back(soft_at(c[i]));
    }
  });
  std::vector<float> w(P, 0.0f);
  on_threads(P, [&](size_t t, size_t nt) {
    for (int p = (int)t; p < P; p += (int)nt) {
      float acc = 0.0f;
      for (int i = 0; i < P; i++)
        for (size_t r = 0; r < nt_used; r++)
          for (float v : terms[r][(size_t)p * P + i]) acc += v;
      w[p] = acc;
    }
  });
  const float scale = (float)(batch * P) / (float)n_data;
  for (int p = 0; p < P; p++) w[p] *= scale;
  return w;
}

// PC: the number of parts when known at compile time (loops over parts unroll), 0 for any
template <int PC> void Partitioner::refine_embed_sweep(std::vector<float> &w) {
  const int P = PC ? PC : n_part;
  std::vector<float> score_v(P), seen_v(P), base_v(P), below_v(P);
  float *score = score_v.data(), *seen = seen_v.data();
  // beta * size of part k, with and without the embedding under decision; refreshed for the two parts of a move
  float *base = base_v.data(), *below = below_v.data();
  for (int k = 0; k < P; k++) {
    base[k] = beta * (float)cnt_embed[k];
    below[k] = beta * (float)(cnt_embed[k] - 1);
  }
  const float per_batch = (float)(batch * P), samples = (float)n_data;
  for (size_t i = 0; i < n_embed; i++) {
    const int32_t *c = &cnt[i * P];
    const int old = res_embed[i];
    int64_t degree = 0;
    for (int j = 0; j < P; j++) degree += c[j];
    for (int k = 0; k < P; k++) score[k] = base[k];
    score[old] = below[old];
    // A part that never uses the embedding sees soft count 0 (soft[0] is exactly 0): subtracting comm * 0 leaves
    // every score as it is, so that part's row of products is skipped; an embedding nobody uses skips all of it.
    if (degree != 0) {
      const double own = (double)soft_at(degree);
      // the reference counts these in float (partition.cc:138-140): above 2^24 such a counter stops growing
      for (int j = 0; j < P; j++) seen[j] = soft_at(std::min<int64_t>(c[j], 1 << 24));
      for (int j = 0; j < P; j++) {
        if (seen[j] != 0.0f) {
          const float *cj = &comm[(size_t)j * P];
          for (int k = 0; k < P; k++) score[k] -= cj[k] * seen[j];
        }
        // partition.cc:149: the literal 0.01 makes this one subtraction a double operation
        score[j] = (float)((double)score[j] - 0.01 * (double)w[j] * own);
      }
    }
    const int to = first_largest(score, P);
    if (to != old) {
      cnt_embed[old]--;
      cnt_embed[to]++;
      res_embed[i] = to;
      for (int k : {old, to}) {
        base[k] = beta * (float)cnt_embed[k];
        below[k] = beta * (float)(cnt_embed[k] - 1);
      }
      if (degree != 0)
        for (int j = 0; j < P; j++) {
          if (c[j] == 0) continue; // soft[0] is 0: the weights would change by 0
          const float t = soft_at(c[j]) * per_batch / samples;
          if (j != to) w[to] += t;
          if (j != old) w[old] -= t;
        }
    }
  }
}

void Partitioner::refine_embed() {
  std::vector<float> w = embed_weight_now();
  switch (n_part) {
  case 2: refine_embed_sweep<2>(w); break;
  case 4: refine_embed_sweep<4>(w); break;
  case 8: refine_embed_sweep<8>(w); break;
  case 16: refine_embed_sweep<16>(w); break;
  default: refine_embed_sweep<0>(w);
  }
}

// cost[i][p]: soft counts, as seen from part i, of the embeddings part p owns, added in ascending embedding id.
// One viewing part per thread.
void Partitioner::communication(float *cost) const {
  const int P = n_part;
  on_threads(P, [&](size_t t, size_t nt) {
    std::vector<float> acc(P);
    for (int i = (int)t; i < P; i += (int)nt) {
      std::fill(acc.begin(), acc.end(), 0.0f);
      for (size_t j = 0; j < n_embed; j++) acc[res_embed[j]] += soft_at(cnt[j * P + i]);
      for (int p = 0; p < P; p++) cost[(size_t)i * P + p] = acc[p];
    }
  });
  const float scale = (float)(batch * P) / (float)n_data;
  for (int i = 0; i < P * P; i++) cost[i] *= scale;
}

namespace {
// partition.cc:188-191: comm * soft^2 * (1/degree + 1/count), every operand widened to double by the double literals
// and std::pow(float, long), rounded to float once.  A float squared is exact in double.
__host__ __device__ inline float priority_value(float comm_ij, float soft_c, int64_t degree, int32_t count) {
  const double sq = (double)soft_c * (double)soft_c;
  return (float)(((double)comm_ij * sq) * ((1.0 / (double)degree) + (1.0 / (double)count)));
}
} // namespace

void Partitioner::priority(float *out) const {
  const int P = n_part;
  on_threads(16, [&](size_t t, size_t nt) {
    const size_t lo = n_embed * t / nt, hi = n_embed * (t + 1) / nt;
    for (size_t j = lo; j < hi; j++) {
      const int32_t *c = &cnt[j * P];
      int64_t degree = 0;
      for (int i = 0; i < P; i++) degree += c[i];
      for (int i = 0; i < P; i++)
        out[(size_t)i * n_embed + j] =
            c[i] == 0 ? 0.0f : priority_value(comm[(size_t)i * P + res_embed[j]], soft_at(c[i]), degree, c[i]);
    }
  });
}

// ---- cache candidates on the GPU ----------------------------------------------------------------------------

namespace {

constexpr int kKeyBlock = 256;

// A float as an unsigned key of the same order, -0 counted as +0; 0 is kept free for "owned by the part".
__device__ inline uint32_t order_key(float v) {
  v += 0.0f;
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : b | 0x80000000u;
}

// One thread per embedding: reads its counter row once and writes the sort key of every part.  PC: the number of
// parts when known at compile time (the row is then read with 16-byte loads), 0 for any.
template <int PC>
__global__ __launch_bounds__(kKeyBlock) void priority_keys(const int32_t *__restrict__ cnt,
                                                           const int32_t *__restrict__ owner,
                                                           const float *__restrict__ soft,
                                                           const float *__restrict__ comm, int n_part, uint32_t n_embed,
                                                           uint32_t n_data, uint32_t *__restrict__ keys) {
  const int P = PC ? PC : n_part;
  const uint32_t j = blockIdx.x * kKeyBlock + threadIdx.x;
  if (j >= n_embed) return;
  const int32_t *c = cnt + (size_t)j * P;
  int32_t row[PC ? PC : 1];
  if (PC) {
    for (int q = 0; q < PC / 4; q++) {
      const int4 v = reinterpret_cast<const int4 *>(c)[q];
      row[4 * q] = v.x, row[4 * q + 1] = v.y, row[4 * q + 2] = v.z, row[4 * q + 3] = v.w;
    }
  }
  int64_t degree = 0;
  for (int i = 0; i < P; i++) degree += PC ? row[i] : c[i];
  const int own = owner[j];
  for (int i = 0; i < P; i++) {
    uint32_t key = 0;
    if (i != own) {
      const int32_t ci = PC ? row[i] : c[i];
      float pr = 0.0f;
      if (ci != 0) pr = priority_value(comm[i * P + own], (uint32_t)ci < n_data ? soft[ci] : 1.0f, degree, ci);
      key = order_key(pr);
    }
    keys[(size_t)i * n_embed + j] = key;
  }
}

// list[q] = the q-th from the end of the ascending order
__global__ __launch_bounds__(kKeyBlock) void emit_reversed(const uint32_t *__restrict__ sorted_pos, uint32_t n,
                                                           uint32_t len, int32_t *__restrict__ list) {
  const uint32_t q = blockIdx.x * kKeyBlock + threadIdx.x;
  if (q < len) list[q] = (int32_t)sorted_pos[n - 1 - q];
}

struct DevMem {
  void *p = nullptr;
  explicit DevMem(size_t bytes) { HCTR_HIP(hipMalloc(&p, std::max<size_t>(bytes, 16))); }
  ~DevMem() { (void)hipFree(p); }
  DevMem(const DevMem &) = delete;
  template <typename T> T *as() const { return (T *)p; }
};

} // namespace

void Partitioner::cache_lists(size_t max_len, int32_t *lists, size_t *lens, float *ms) const {
  const int P = n_part;
  HCTR_CHECK(lists && lens, "partition: null argument");
  HCTR_CHECK(n_embed < (1ull << 31), "partition: too many embeddings");
  const uint32_t n = (uint32_t)n_embed;
  const size_t keep = std::min<size_t>(max_len, n_embed);
  DevMem d_cnt(cnt.size() * 4), d_owner(n_embed * 4), d_soft(soft.size() * 4), d_comm(comm.size() * 4);
  DevMem d_keys((size_t)P * n * 4), k0((size_t)n * 4), k1((size_t)n * 4), v0((size_t)n * 4), v1((size_t)n * 4),
      pos((size_t)n * 4), d_lists((size_t)P * keep * 4);
  SortScratch sc;
  DevMem d_ws(sort_scratch_words(n) * 4);
  sc.words = d_ws.as<uint32_t>();
  sc.n_cap = n;
  hipStream_t s = nullptr;
  HCTR_HIP(hipMemcpyAsync(d_cnt.p, cnt.data(), cnt.size() * 4, hipMemcpyHostToDevice, s));
  HCTR_HIP(hipMemcpyAsync(d_owner.p, res_embed.data(), n_embed * 4, hipMemcpyHostToDevice, s));
  HCTR_HIP(hipMemcpyAsync(d_soft.p, soft.data(), soft.size() * 4, hipMemcpyHostToDevice, s));
  HCTR_HIP(hipMemcpyAsync(d_comm.p, comm.data(), comm.size() * 4, hipMemcpyHostToDevice, s));
  hipEvent_t e0, e1;
  HCTR_HIP(hipEventCreate(&e0));
  HCTR_HIP(hipEventCreate(&e1));
  HCTR_HIP(hipEventRecord(e0, s));
  auto keys_kernel = priority_keys<0>;
  if (P == 4) keys_kernel = priority_keys<4>;
  if (P == 8) keys_kernel = priority_keys<8>;
  if (P == 16) keys_kernel = priority_keys<16>;
  hipLaunchKernelGGL(keys_kernel, dim3(div_up(n, kKeyBlock)), dim3(kKeyBlock), 0, s, d_cnt.as<int32_t>(),
                     d_owner.as<int32_t>(), d_soft.as<float>(), d_comm.as<float>(), P, n, (uint32_t)n_data,
                     d_keys.as<uint32_t>());
  HCTR_HIP(hipGetLastError());
  for (int i = 0; i < P; i++) {
    const uint32_t *sorted_keys;
    radix_sort_positions<uint32_t>(s, d_keys.as<uint32_t>() + (size_t)i * n, n, 32, k0.as<uint32_t>(),
                                   k1.as<uint32_t>(), v0.as<uint32_t>(), v1.as<uint32_t>(), pos.as<uint32_t>(), sc,
                                   &sorted_keys);
    lens[i] = std::min<size_t>(keep, n_embed - (size_t)cnt_embed[i]);
    if (lens[i]) {
      hipLaunchKernelGGL(emit_reversed, dim3(div_up(lens[i], kKeyBlock)), dim3(kKeyBlock), 0, s, pos.as<uint32_t>(), n,
                         (uint32_t)lens[i], d_lists.as<int32_t>() + (size_t)i * keep);
      HCTR_HIP(hipGetLastError());
    }
  }
  HCTR_HIP(hipEventRecord(e1, s));
  for (int i = 0; i < P; i++)
    if (lens[i])
      HCTR_HIP(hipMemcpyAsync(lists + (size_t)i * max_len, d_lists.as<int32_t>() + (size_t)i * keep, lens[i] * 4,
                              hipMemcpyDeviceToHost, s));
  HCTR_HIP(hipStreamSynchronize(s));
  float t = 0.f;
  HCTR_HIP(hipEventElapsedTime(&t, e0, e1));
  if (ms) *ms = t;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
}

} // namespace hctr
