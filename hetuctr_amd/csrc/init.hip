// Table initialisation kernels: seeded value initialisers, fills, and the id -> resident-offset directory.
// Reference: csrc/utils/initializer.cu:11-103 (Zero / Normal / Uniform / TruncatedNormal through
// thrust::minstd_rand with discard(n) per element) and csrc/core/table_initialize.cu:84-112.
//
// The reference keeps id -> offset in a hash map (csrc/cudf/concurrent_unordered_map.cuh:564-587); only
// the result of find() is observable.  Ids are dense (root_arr has one entry per id), so here the map is
// a plain array indexed by id: one 4-byte load per lookup, no probing, 4 bytes per id of HBM.
#include "kernels.h"

namespace hctr {
namespace {

constexpr int kBlock = 256;
constexpr int kPerThread = 16;
constexpr uint64_t kA = 48271ull, kM = 2147483647ull;

__device__ __forceinline__ uint32_t lcg_pow(uint64_t e) {
  uint64_t r = 1, b = kA;
  while (e) {
    if (e & 1) r = r * b % kM;
    b = b * b % kM;
    e >>= 1;
  }
  return (uint32_t)r;
}
__device__ __forceinline__ uint32_t lcg_next(uint32_t x) { return (uint32_t)((uint64_t)x * kA % kM); }

// thrust::uniform_real_distribution<float>: (x - min) / (1 + (max - min)) * (b - a) + a, min = 1, max = m - 1
__device__ __forceinline__ float draw_uniform(uint32_t x, float a, float b) {
  float r = (float)(x - 1u);
  r /= (1.0f + (float)(uint32_t)(kM - 2));
  return __fmaf_rn(r, b - a, a);
}
// thrust's direct-sampling normal for device compilers: mean + sigma * (-+sqrt 2) * erfcinv(2p)
__device__ __forceinline__ float draw_normal(uint32_t x, float mean, float stddev) {
  const uint32_t range = (uint32_t)(kM - 2);
  const float S1 = (float)(1.0 / (double)range);
  const float S2 = S1 / 2;
  float S3 = -1.4142135623730950488f;
  uint32_t u = x - 1u;
  if (u > range / 2) {
    u = range - u;
    S3 = -S3;
  }
  const float p = __fmaf_rn((float)u, S1, S2);
  return __fmaf_rn(stddev * S3, erfcinvf(2 * p), mean);
}

__global__ __launch_bounds__(kBlock) void init_values(embed_t *__restrict__ out, size_t len, int type, float a,
                                                      float b, uint32_t state0) {
  const size_t n0 = ((size_t)blockIdx.x * kBlock + threadIdx.x) * kPerThread;
  if (n0 >= len) return;
  // element n draws x_{n+1} = state0 * 48271^(n+1) mod m
  uint32_t x = (uint32_t)((uint64_t)lcg_pow(n0 + 1) * state0 % kM);
  for (int k = 0; k < kPerThread && n0 + k < len; k++) {
    float v;
    if (type == 2) v = draw_uniform(x, a, b);
    else if (type == 1) v = draw_normal(x, a, b);
    else {
      uint32_t y = x;
      for (;;) { // redraw with rng.seed(rng()) until inside two sigma (initializer.cu:60-67)
        v = draw_normal(y, a, b);
        y = lcg_next(y);
        if (!(v > a + 2 * b || v < a - 2 * b)) break;
        y = lcg_next(y);
      }
    }
    out[n0 + k] = v;
    x = lcg_next(x);
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void fill(T *__restrict__ p, size_t n, T v) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) p[i] = v;
}

__global__ __launch_bounds__(kBlock) void build_directory(const index_t *__restrict__ store_ids, uint32_t n,
                                                          slot_t *__restrict__ slot) {
  const uint32_t o = blockIdx.x * kBlock + threadIdx.x;
  if (o < n) slot[store_ids[o]] = (slot_t)o;
}

} // namespace

void launch_init_values(hipStream_t s, embed_t *out, size_t len, int type, float a, float b, unsigned seed) {
  if (!len) return;
  if (type == 0) {
    HCTR_HIP(hipMemsetAsync(out, 0, len * sizeof(embed_t), s));
    return;
  }
  uint32_t st = (uint32_t)(seed % kM);
  if (st == 0) st = 1; // an engine with increment 0 replaces state 0 by 1
  const size_t threads = (len + kPerThread - 1) / kPerThread;
  hipLaunchKernelGGL(init_values, dim3(div_up(threads, kBlock)), dim3(kBlock), 0, s, out, len, type, a, b, st);
  HCTR_HIP(hipGetLastError());
}

void launch_fill_i64(hipStream_t s, version_t *p, size_t n, version_t v) {
  if (!n) return;
  hipLaunchKernelGGL(fill<version_t>, dim3((unsigned)std::min<size_t>(div_up(n, kBlock), 8192)), dim3(kBlock), 0, s, p, n, v);
  HCTR_HIP(hipGetLastError());
}

void launch_fill_i32(hipStream_t s, int32_t *p, size_t n, int32_t v) {
  if (!n) return;
  hipLaunchKernelGGL(fill<int32_t>, dim3((unsigned)std::min<size_t>(div_up(n, kBlock), 8192)), dim3(kBlock), 0, s, p, n, v);
  HCTR_HIP(hipGetLastError());
}

void launch_build_directory(hipStream_t s, const index_t *store_ids, uint32_t n_stored, slot_t *slot) {
  if (!n_stored) return;
  hipLaunchKernelGGL(build_directory, dim3(div_up(n_stored, kBlock)), dim3(kBlock), 0, s, store_ids, n_stored, slot);
  HCTR_HIP(hipGetLastError());
}

} // namespace hctr
