// Shared declarations of the HIP library: scalar types, error handling, small device helpers.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>

namespace hctr {

// csrc/core/types.h:12-28 of the reference: the types that cross the boundary
typedef float embed_t;
typedef long long version_t;
typedef long long index_t;
typedef unsigned char worker_t;
constexpr index_t kInvalidIndex = -1;
constexpr version_t kInvalidVersion = (version_t)0x8000000000000000ULL; // numeric_limits<long long>::min()

// Inside the library resident offsets and batch positions are 32-bit: a shard holds < 2^31 rows and a
// batch < 2^32 keys.  -1 marks "not resident".
typedef int32_t slot_t;
constexpr slot_t kNoSlot = -1;

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

#define HCTR_HIP(expr)                                                                              \
  do {                                                                                              \
    hipError_t e__ = (expr);                                                                        \
    if (e__ != hipSuccess)                                                                          \
      throw ::hctr::Error(std::string(#expr) + " failed: " + hipGetErrorString(e__) + " (" + __FILE__ + \
                          ":" + std::to_string(__LINE__) + ")");                                   \
  } while (0)

#define HCTR_CHECK(cond, msg)                                   \
  do {                                                          \
    if (!(cond)) throw ::hctr::Error(std::string("hetuCTR: ") + (msg)); \
  } while (0)

inline unsigned div_up(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

constexpr int kWave = 64;

// ---- device helpers ---------------------------------------------------------------------------
// a load of data that nothing reads again soon: it should not push other lines out of the caches
template <typename T> __device__ __forceinline__ T load_once(const T *p) { return __builtin_nontemporal_load(p); }

__device__ __forceinline__ unsigned lane_id() { return __lane_id(); }

// inclusive scan over the 64 lanes of a wave
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    uint32_t n = __shfl_up(v, d, kWave);
    if ((int)lane_id() >= d) v += n;
  }
  return v;
}

// Exclusive scan of one value per thread over a block of NT threads (NT multiple of 64, <= 1024).
// `total` receives the block sum.  `smem` needs NT/64 + 1 words.  Contains __syncthreads.
template <int NT>
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t *smem, uint32_t &total) {
  constexpr int NW = NT / kWave;
  const int w = threadIdx.x / kWave;
  uint32_t inc = wave_inclusive_scan(v);
  if (lane_id() == kWave - 1) smem[w] = inc;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t run = 0;
#pragma unroll
    for (int i = 0; i < NW; i++) {
      uint32_t t = smem[i];
      smem[i] = run;
      run += t;
    }
    smem[NW] = run;
  }
  __syncthreads();
  uint32_t res = inc - v + smem[w];
  total = smem[NW];
  __syncthreads();
  return res;
}

} // namespace hctr
