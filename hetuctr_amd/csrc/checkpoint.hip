// Checkpoint of one shard: the resident rows with their versions and, for cached rows, the pending gradients and
// update counters, written to and read back from one file per shard.  The reference keeps all of this in device
// memory only (csrc/core/hetu_gpu_table.h:38-70) and has no way to save it; a caller that restarts a job needs one.
//
// File layout (little endian, no padding between the parts):
//   Header (below) | store_ids int64[n_stored] | emb float[n_stored][width] | ver int64[n_stored] |
//   pend float[n_cached][width] | upd int64[n_cached]
// store_ids is the resident layout (cached ids first, then owned ids): a file only loads into a table built from
// the same root_arr / storage_arr.
#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <vector>

#include <sys/stat.h>

#include "table.h"

namespace hctr {
namespace {

struct Header {
  char magic[8]; // "HCTRCKP1"
  uint32_t rank, nrank, width, reserved;
  uint64_t length, n_stored, n_cached;
  int64_t pull_bound, push_bound;
};

constexpr size_t kStageBytes = 32u << 20; // pinned staging area the device data travels through

struct Staging {
  void *p = nullptr;
  Staging() { HCTR_HIP(hipHostMalloc(&p, kStageBytes, hipHostMallocDefault)); }
  ~Staging() {
    if (p) (void)hipHostFree(p);
  }
};

struct File {
  FILE *f;
  std::string path;
  File(const char *p, const char *mode) : f(fopen(p, mode)), path(p) {
    HCTR_CHECK(f != nullptr, "cannot open " + path + ": " + strerror(errno));
  }
  ~File() {
    if (f) fclose(f);
  }
  void close() { // a failed close loses buffered data: it is an error of the write, not something to ignore
    FILE *g = f;
    f = nullptr;
    HCTR_CHECK(fclose(g) == 0, "cannot close " + path + ": " + strerror(errno));
  }
  uint64_t size() {
    struct stat sb;
    HCTR_CHECK(fstat(fileno(f), &sb) == 0, "cannot stat " + path + ": " + strerror(errno));
    return (uint64_t)sb.st_size;
  }
  void write(const void *d, size_t n) { HCTR_CHECK(fwrite(d, 1, n, f) == n, "short write to " + path); }
  void read(void *d, size_t n) { HCTR_CHECK(fread(d, 1, n, f) == n, "short read from " + path + " (truncated file?)"); }
};

void device_to_file(File &out, const void *dev, size_t bytes, Staging &st, hipStream_t s) {
  for (size_t done = 0; done < bytes; done += kStageBytes) {
    const size_t n = std::min(kStageBytes, bytes - done);
    HCTR_HIP(hipMemcpyAsync(st.p, (const char *)dev + done, n, hipMemcpyDeviceToHost, s));
    HCTR_HIP(hipStreamSynchronize(s));
    out.write(st.p, n);
  }
}

void file_to_device(File &in, void *dev, size_t bytes, Staging &st, hipStream_t s) {
  for (size_t done = 0; done < bytes; done += kStageBytes) {
    const size_t n = std::min(kStageBytes, bytes - done);
    in.read(st.p, n);
    HCTR_HIP(hipMemcpyAsync((char *)dev + done, st.p, n, hipMemcpyHostToDevice, s));
    HCTR_HIP(hipStreamSynchronize(s));
  }
}

// the file's copy of an array against the device's, piece by piece
void compare_with_device(File &in, const void *dev, size_t bytes, Staging &st, hipStream_t s, const char *what) {
  std::vector<char> host(std::min(kStageBytes, std::max<size_t>(bytes, 1)));
  for (size_t done = 0; done < bytes; done += kStageBytes) {
    const size_t n = std::min(kStageBytes, bytes - done);
    in.read(host.data(), n);
    HCTR_HIP(hipMemcpyAsync(st.p, (const char *)dev + done, n, hipMemcpyDeviceToHost, s));
    HCTR_HIP(hipStreamSynchronize(s));
    HCTR_CHECK(memcmp(host.data(), st.p, n) == 0, std::string("checkpoint: ") + what + " differ from the table's");
  }
}

} // namespace

void Shard::save(const char *path) {
  HCTR_CHECK(path && *path, "null path");
  HCTR_HIP(hipSetDevice(cfg.device_id));
  group->flush_index();
  hipStream_t s = group->stream;
  HCTR_HIP(hipStreamSynchronize(s));
  Header h;
  memset(&h, 0, sizeof h);
  memcpy(h.magic, "HCTRCKP1", 8);
  h.rank = cfg.rank, h.nrank = cfg.nrank, h.width = tv.width;
  h.length = tv.id_max, h.n_stored = tv.n_stored, h.n_cached = tv.n_cached;
  h.pull_bound = tv.pull_bound, h.push_bound = tv.push_bound;
  const size_t S = tv.n_stored, C = tv.n_cached, W = tv.width;
  Staging st;
  // written beside the target and renamed over it when it is complete and closed: a crash or a full disk in the
  // middle leaves the checkpoint that was there before
  const std::string tmp = std::string(path) + ".tmp";
  try {
    File out(tmp.c_str(), "wb");
    out.write(&h, sizeof h);
    device_to_file(out, store_ids.p, S * sizeof(index_t), st, s);
    device_to_file(out, emb.p, S * W * sizeof(embed_t), st, s);
    device_to_file(out, ver.p, S * sizeof(version_t), st, s);
    device_to_file(out, pend.p, C * W * sizeof(embed_t), st, s);
    device_to_file(out, upd.p, C * sizeof(version_t), st, s);
    HCTR_CHECK(fflush(out.f) == 0, "cannot flush " + out.path + ": " + strerror(errno));
    out.close();
    HCTR_CHECK(rename(tmp.c_str(), path) == 0, "cannot rename " + tmp + " to " + path + ": " + strerror(errno));
  } catch (...) {
    (void)remove(tmp.c_str());
    throw;
  }
}

void Shard::load(const char *path) {
  HCTR_CHECK(path && *path, "null path");
  HCTR_HIP(hipSetDevice(cfg.device_id));
  group->flush_index();
  hipStream_t s = group->stream;
  HCTR_HIP(hipStreamSynchronize(s));
  File in(path, "rb");
  Header h;
  in.read(&h, sizeof h);
  HCTR_CHECK(memcmp(h.magic, "HCTRCKP1", 8) == 0, "not a hetuCTR checkpoint: " + in.path);
  HCTR_CHECK(h.rank == (uint32_t)cfg.rank && h.nrank == (uint32_t)cfg.nrank, "checkpoint of another rank / group size");
  HCTR_CHECK(h.width == tv.width && h.length == tv.id_max, "checkpoint of a table with another width / length");
  HCTR_CHECK(h.n_stored == tv.n_stored && h.n_cached == tv.n_cached,
             "checkpoint of a shard with other resident rows (storage_arr differs)");
  const size_t S = tv.n_stored, C = tv.n_cached, W = tv.width;
  // all or nothing: the length of the file is checked before the first array of the table is overwritten
  const uint64_t want = sizeof(Header) + (uint64_t)S * sizeof(index_t) + (uint64_t)S * W * sizeof(embed_t) +
                        (uint64_t)S * sizeof(version_t) + (uint64_t)C * W * sizeof(embed_t) + (uint64_t)C * sizeof(version_t);
  const uint64_t have = in.size();
  HCTR_CHECK(have >= want, "checkpoint is shorter than the table (truncated file?): " + in.path);
  HCTR_CHECK(have == want, "checkpoint is longer than the table: " + in.path);
  Staging st;
  compare_with_device(in, store_ids.p, S * sizeof(index_t), st, s, "the resident ids");
  file_to_device(in, emb.p, S * W * sizeof(embed_t), st, s);
  file_to_device(in, ver.p, S * sizeof(version_t), st, s);
  file_to_device(in, pend.p, C * W * sizeof(embed_t), st, s);
  file_to_device(in, upd.p, C * sizeof(version_t), st, s);
  // the batches in flight belong to the run that wrote the file, not to this one: start from empty ones
  for (Batch *b : {&cur, &prev}) {
    b->n = 0;
    b->U = 0;
    b->idx_map_valid = false;
    b->planned = false;
    b->clear(s, cfg.nrank);
    std::fill(b->send_cnt.begin(), b->send_cnt.end(), 0);
    std::fill(b->recv_cnt.begin(), b->recv_cnt.end(), 0);
    std::fill(b->push_cnt.begin(), b->push_cnt.end(), 0);
    std::fill(b->pushrecv_cnt.begin(), b->pushrecv_cnt.end(), 0);
  }
  prev_active = false;
  HCTR_HIP(hipStreamSynchronize(s));
}

} // namespace hctr
