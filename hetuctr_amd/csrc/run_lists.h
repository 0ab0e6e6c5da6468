// The run lists of a batch for the push that sums its gradients one step later: runs longer than kLongRun by length
// class, runs of medium length in one list (the lists' layout is with BatchView in kernels.h).  They are built after the
// unique pass by whichever kernel comes next anyway -- the gather of the step, whose first blocks take a chunk of unique
// ranks each before their own work -- or by a launch of their own where no gather follows.
#pragma once
#include "kernels.h"

namespace hctr {

constexpr int kRunListBlock = 256;           // unique ranks per chunk = threads of the block that lists them
constexpr int kRunLists = kLongBuckets + 1;  // length classes of long runs, then the medium list

// Chunk `chunk` of the unique ranks, one rank per thread of a kRunListBlock-thread block.  Atomics on one address are
// served one after the other, so a block reserves its list entries with ONE atomic per list: entries are counted and
// placed inside the block through LDS first.  cnt / base: kRunLists LDS words each.  Contains barriers: every thread of
// the block calls it (the chunk is the same for all of them).
__device__ __forceinline__ void list_runs_chunk(const BatchView &b, uint32_t chunk, uint32_t *cnt, uint32_t *base) {
  const uint32_t U = *b.d_U;
  if (chunk * kRunListBlock >= U) return; // whole chunk past the last unique key
  const uint32_t u = chunk * kRunListBlock + threadIdx.x;
  if (threadIdx.x < kRunLists) cnt[threadIdx.x] = 0;
  __syncthreads();
  const bool valid = u < U;
  const uint32_t len = valid ? b.run_start[u + 1] - b.run_start[u] : 0u;
  int list = -1;
  if (len > kLongRun) list = long_bucket(len);
  else if (len > kTinyRun) list = kLongBuckets;
  uint32_t local = 0;
  if (list >= 0) local = atomicAdd(&cnt[list], 1u); // LDS atomic: the order inside a list does not matter
  __syncthreads();
  if (threadIdx.x < kRunLists && cnt[threadIdx.x])
    base[threadIdx.x] = atomicAdd(&b.d_nlong[threadIdx.x < kLongBuckets ? threadIdx.x : kMedCount], cnt[threadIdx.x]);
  __syncthreads();
  if (list >= 0) {
    if (list < kLongBuckets)
      b.long_list[(size_t)list * b.long_cap + base[list] + local] = make_uint4(u, b.run_start[u], len, (uint32_t)b.uoff[u]);
    else b.med_list[base[list] + local] = u;
  }
  __syncthreads(); // cnt / base are free again
}

} // namespace hctr
