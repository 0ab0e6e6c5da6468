// Offline partitioner: assigns samples and embedding rows to parts so that few rows cross parts, and ranks, per
// part, the rows it does not own by how much caching them would save.  Same results as the reference's
// PartitionStruct (csrc/partition/partition.h:8-30, partition.cc:26-194) run without OpenMP threads.
//
// Layout differs from the reference: one counter table cnt[embedding][part] (a part's view of an embedding is one
// 4*n_part-byte row, one cache line for 8 parts) replaces the per-part arrays, and the transposed sample list per
// embedding is not built at all, because what the embedding sweep counts with it is that same row.
#pragma once
#include <memory>
#include <utility>
#include <vector>

#include "common.h"

namespace hctr {

// std::allocator whose value-less construct leaves the memory as it is (resize() without the zero fill)
template <typename T> struct LeaveUninit : std::allocator<T> {
  template <typename U> struct rebind {
    using other = LeaveUninit<U>;
  };
  template <typename U, typename... A> void construct(U *p, A &&...a) {
    if constexpr (sizeof...(A) == 0)
      ::new ((void *)p) U;
    else
      ::new ((void *)p) U(std::forward<A>(a)...);
  }
};

class Partitioner {
public:
  Partitioner(const int32_t *data, size_t n_data, size_t n_slot, const float *comm_mat, int n_part, int batch_size,
              unsigned seed);

  void refine_data();                    // partition.cc:89-120
  void refine_embed();                   // partition.cc:122-166
  void communication(float *cost) const; // partition.cc:168-181, cost[n_part][n_part]
  void priority(float *out) const;       // partition.cc:183-194, out[n_part][n_embed]
  // Per part the embeddings it does not own, by descending priority, equal priorities by descending id
  // (experimental/partition.py:53-57); at most max_len per part into lists[part * max_len ..], lens[part] of them.
  // Computed on the GPU; ms receives the device time of the kernels.
  void cache_lists(size_t max_len, int32_t *lists, size_t *lens, float *ms) const;

  int n_part, batch;
  size_t n_data, n_slot, n_embed;
  std::vector<int32_t> res_data, res_embed, cnt_data, cnt_embed;

private:
  float soft_at(int64_t i) const { return i < (int64_t)n_data ? soft[i] : 1.0f; }
  std::vector<float> embed_weight_now() const;
  template <int PC> void refine_data_sweep();
  template <int PC> void refine_embed_sweep(std::vector<float> &w);

  float alpha, beta;
  std::vector<int32_t> data; // [n_data][n_slot]
  std::vector<int32_t, LeaveUninit<int32_t>> cnt; // [n_embed][n_part]: samples of the part using the embedding, once per slot
  std::vector<float> soft;   // [n_data]
  std::vector<float> dsoft;  // [n_data + 1]: soft_at(i + 1) - soft_at(i); the last entry (and all beyond) 0
  std::vector<float> comm;   // [n_part][n_part], comm[i][j] = cost for part i of a row owned by part j
  std::vector<float> comm_t; // transposed
};

} // namespace hctr
