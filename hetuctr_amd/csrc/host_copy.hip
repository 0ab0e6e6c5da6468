// Pageable host memory -> device through a pinned staging buffer filled by a crew of threads.  Host code only.
#include "host_copy.h"

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace hctr {
namespace {

constexpr size_t kPiece = 128 << 10;      // bytes a thread copies at a time
constexpr size_t kCrewFrom = 1 << 20;     // smaller copies are done by the calling thread alone
constexpr size_t kTransferStep = 1 << 20; // a transfer is issued for every this many contiguous bytes ready
constexpr int kSpinMicros = 100;          // an idle crew thread polls this long for the next copy before it sleeps

// one copy: pieces are handed out through `next`, a finished piece sets its flag
struct Job {
  const unsigned char *src;
  unsigned char *dst;
  size_t bytes, pieces; // of the source
  bool narrow;          // the source is 64-bit ids, the staging buffer gets 32-bit ones
  std::atomic<size_t> next{0};
  std::unique_ptr<std::atomic<unsigned char>[]> done;

  Job(const void *s, void *d, size_t n, bool narrow_ids)
      : src((const unsigned char *)s), dst((unsigned char *)d), bytes(n), pieces((n + kPiece - 1) / kPiece), narrow(narrow_ids) {
    done.reset(new std::atomic<unsigned char>[pieces]);
    for (size_t i = 0; i < pieces; i++) done[i].store(0, std::memory_order_relaxed);
  }
  // bytes of the staging buffer the first `p` pieces fill
  size_t staged(size_t p) const { return std::min(p * kPiece, bytes) / (narrow ? 2 : 1); }
  bool take_piece() {
    const size_t i = next.fetch_add(1, std::memory_order_relaxed);
    if (i >= pieces) return false;
    const size_t lo = i * kPiece, len = std::min(kPiece, bytes - lo);
    if (narrow) narrow_ids(dst + lo / 2, src + lo, len / sizeof(int64_t));
    else std::memcpy(dst + lo, src + lo, len);
    done[i].store(1, std::memory_order_release);
    return true;
  }
  // an id that does not fit 32 bits (negative ones included) becomes 0xffffffff
  static void narrow_ids(unsigned char *to, const unsigned char *from, size_t n) {
    const uint64_t *__restrict__ in = (const uint64_t *)from;
    uint32_t *__restrict__ out = (uint32_t *)to;
    for (size_t k = 0; k < n; k++) {
      const uint64_t v = in[k];
      out[k] = (v >> 32) ? 0xffffffffu : (uint32_t)v;
    }
  }
};

// The crew: threads that sleep until a job is posted.  A thread that wakes late finds the job's pieces handed out
// and goes back to sleep; it keeps the job alive through its shared_ptr, so the poster never waits for the crew.
class Crew {
 public:
  explicit Crew(int workers) {
    for (int i = 0; i < workers; i++) threads_.emplace_back([this] { run(); });
  }
  ~Crew() {
    {
      std::lock_guard<std::mutex> g(mu_);
      stop_ = true;
      seq_.fetch_add(1, std::memory_order_release);
    }
    cv_.notify_all();
    for (std::thread &t : threads_) t.join();
  }
  void post(const std::shared_ptr<Job> &job) {
    {
      std::lock_guard<std::mutex> g(mu_);
      job_ = job;
      seq_.fetch_add(1, std::memory_order_release);
    }
    cv_.notify_all();
  }
  size_t workers() const { return threads_.size(); }

 private:
  void run() {
    uint64_t seen = 0;
    for (;;) {
      // poll for a while (the next batch usually follows within a training step), then sleep
      const auto until = std::chrono::steady_clock::now() + std::chrono::microseconds(kSpinMicros);
      while (seq_.load(std::memory_order_acquire) == seen && std::chrono::steady_clock::now() < until) __builtin_ia32_pause();
      std::shared_ptr<Job> job;
      {
        std::unique_lock<std::mutex> g(mu_);
        cv_.wait(g, [&] { return seq_.load(std::memory_order_acquire) != seen; });
        seen = seq_.load(std::memory_order_acquire);
        if (stop_) return;
        job = job_;
      }
      if (job)
        while (job->take_piece()) {
        }
    }
  }
  std::mutex mu_;
  std::condition_variable cv_;
  std::atomic<uint64_t> seq_{0};
  std::shared_ptr<Job> job_;
  bool stop_ = false;
  std::vector<std::thread> threads_;
};

Crew &crew() {
  static Crew c(host_copy_threads() - 1);
  return c;
}

} // namespace

int host_copy_threads() {
  static const int n = [] {
    const char *e = std::getenv("HETUCTR_COPY_THREADS");
    int v = e ? std::atoi(e) : 8;
    return v < 1 ? 1 : (v > 64 ? 64 : v);
  }();
  return n;
}

HostStager::~HostStager() {
  if (sent_) {
    (void)hipEventSynchronize(sent_);
    (void)hipEventDestroy(sent_);
  }
  if (pinned_) (void)hipHostFree(pinned_);
}

void HostStager::copy(void *dst, const void *src, size_t bytes, hipStream_t s, bool narrow_ids) {
  if (!bytes) return;
  // the transfers of the call before read the staging buffer: they have normally completed long ago
  if (sent_) HCTR_HIP(hipEventSynchronize(sent_));
  else HCTR_HIP(hipEventCreateWithFlags(&sent_, hipEventDisableTiming));
  if (bytes > cap_) {
    if (pinned_) HCTR_HIP(hipHostFree(pinned_));
    pinned_ = nullptr;
    cap_ = 0;
    const size_t want = bytes + bytes / 4;
    HCTR_HIP(hipHostMalloc((void **)&pinned_, want, hipHostMallocDefault));
    cap_ = want;
  }
  auto job = std::make_shared<Job>(src, pinned_, bytes, narrow_ids);
  const bool alone = bytes < kCrewFrom || host_copy_threads() == 1;
  if (!alone) crew().post(job);
  // this thread copies pieces too, and between them sends off what is ready: pieces 0..ready-1 are in the staging buffer
  size_t ready = 0, sent = 0; // pieces / bytes of the staging buffer
  auto count_ready = [&] {
    while (ready < job->pieces && job->done[ready].load(std::memory_order_acquire)) ready++;
  };
  auto send = [&](bool all) {
    const size_t have = job->staged(ready);
    if (have - sent >= kTransferStep || (all && have > sent)) {
      HCTR_HIP(hipMemcpyAsync((unsigned char *)dst + sent, pinned_ + sent, have - sent, hipMemcpyHostToDevice, s));
      sent = have;
    }
  };
  auto stage = [&](bool sending) { // until every piece is in the staging buffer: nobody reads `src` after that
    while (job->take_piece()) {
      count_ready();
      if (sending) send(false);
    }
    while (count_ready(), ready < job->pieces) { // pieces other threads are still copying
      if (sending) send(false);
      __builtin_ia32_pause();
    }
  };
  try {
    stage(true);
    send(true);
    HCTR_HIP(hipEventRecord(sent_, s));
  } catch (...) {
    stage(false); // a failed transfer must not leave the crew reading the caller's buffer after this call
    throw;
  }
}

} // namespace hctr
