// Batch sampling from a click log that lives in HBM: what the reference's benchmark does on the host with numpy
// (tests/benchmark.py:19-23: data[idx].flatten() for random sample rows idx of an int64 [samples][fields] array)
// as one kernel, so that the ids handed to preprocess are already on the device.
#include "kernels.h"

namespace hctr {
namespace {

constexpr int kBlock = 256;

// one thread per output id: keys_out[r * fields + f] = log[rows[r] * fields + f]
__global__ __launch_bounds__(kBlock) void sample_rows(const index_t *__restrict__ log, uint64_t n_samples,
                                                      uint32_t fields, const index_t *__restrict__ rows,
                                                      uint64_t n_out, index_t *__restrict__ keys_out,
                                                      uint32_t *__restrict__ err) {
  const uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_out) return;
  const uint64_t r = i / fields, f = i % fields;
  const uint64_t row = (uint64_t)rows[r];
  if (row >= n_samples) { // also catches negative row numbers
    atomicOr(err, 1u);
    keys_out[i] = 0;
    return;
  }
  keys_out[i] = log[row * fields + f];
}

} // namespace

void launch_sample_rows(hipStream_t s, const index_t *log, uint64_t n_samples, uint32_t fields, const index_t *rows,
                        uint64_t n_rows, index_t *keys_out, uint32_t *err) {
  const uint64_t n_out = n_rows * fields;
  if (!n_out) return;
  HCTR_CHECK(n_out < ((uint64_t)1 << 40), "sample_rows: too many ids for one launch");
  hipLaunchKernelGGL(sample_rows, dim3((unsigned)((n_out + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, log, n_samples, fields,
                     rows, n_out, keys_out, err);
  HCTR_HIP(hipGetLastError());
}

} // namespace hctr
