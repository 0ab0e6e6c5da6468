// Python module `hetuCTR`: the reference's python surface (csrc/pybind/pybind.cu:42-79, container.h:12-37)
// on top of the C ABI of libhetuctr_hip.so.  Host-only C++; everything GPU-side happens behind hctr_* calls.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>

#include <condition_variable>
#include <deque>
#include <functional>
#include <future>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <thread>

#include "hetuctr_hip.h"

namespace py = pybind11;

namespace {

// csrc/utils/initializer.h:8-25
enum class InitType { kZero = HCTR_INIT_ZERO, kNormal = HCTR_INIT_NORMAL, kUniform = HCTR_INIT_UNIFORM,
                      kTruncatedNormal = HCTR_INIT_TRUNCATED_NORMAL };
struct Initializer {
  Initializer(InitType t, float a_, float b_) : type(t), a(a_), b(b_) {}
  InitType type;
  float a, b;
};

[[noreturn]] void raise_last() { throw std::runtime_error(hctr_last_error()); }

// One worker thread, first in first out: what the reference's ThreadPool(1) gives the async_* calls
// (csrc/pybind/container.h:24-34, csrc/utils/thread_pool.h:21-36).
class SerialWorker {
 public:
  SerialWorker() : thread_([this] { loop(); }) {}
  ~SerialWorker() {
    {
      std::lock_guard<std::mutex> lk(mu_);
      stop_ = true;
    }
    cv_.notify_all();
    thread_.join();
  }
  std::shared_future<void> enqueue(std::function<void()> f) {
    auto task = std::make_shared<std::packaged_task<void()>>(std::move(f));
    std::shared_future<void> fut = task->get_future().share();
    {
      std::lock_guard<std::mutex> lk(mu_);
      if (stop_) throw std::runtime_error("enqueue on stopped worker");
      q_.emplace_back([task] { (*task)(); });
    }
    cv_.notify_one();
    return fut;
  }

 private:
  void loop() {
    for (;;) {
      std::function<void()> f;
      {
        std::unique_lock<std::mutex> lk(mu_);
        cv_.wait(lk, [this] { return stop_ || !q_.empty(); });
        if (q_.empty()) return; // stop requested and everything queued has run
        f = std::move(q_.front());
        q_.pop_front();
      }
      f();
    }
  }
  std::mutex mu_;
  std::condition_variable cv_;
  std::deque<std::function<void()>> q_;
  bool stop_ = false;
  std::thread thread_;
};

// csrc/pybind/container.h:12-37
class TableContainer {
 public:
  TableContainer(int rank, int nrank, int device_id, const std::string &ip, int port, size_t length, size_t width,
                 long long pull_bound, long long push_bound, py::array_t<uint8_t> root_arr,
                 py::array_t<long long> storage_arr, const Initializer &init, float learning_rate, int verbose) {
    // csrc/pybind/pybind.h:51-56
    if (!root_arr.attr("flags").attr("c_contiguous").cast<bool>())
      throw std::runtime_error("Array not continuous in C: root_id_arr");
    if (!storage_arr.attr("flags").attr("c_contiguous").cast<bool>())
      throw std::runtime_error("Array not continuous in C: storage_id_arr");
    if ((size_t)root_arr.size() != length) throw std::runtime_error("root_arr must hold `length` entries");
    hctr_config cfg{};
    cfg.rank = rank;
    cfg.nrank = nrank;
    cfg.device_id = device_id;
    cfg.ip = ip.c_str();
    cfg.port = port;
    cfg.length = length;
    cfg.width = width;
    cfg.pull_bound = pull_bound;
    cfg.push_bound = push_bound;
    cfg.init_type = (int)init.type;
    cfg.init_a = init.a;
    cfg.init_b = init.b;
    cfg.learning_rate = learning_rate;
    cfg.verbose = verbose;
    const uint8_t *root = root_arr.data();
    const int64_t *storage = reinterpret_cast<const int64_t *>(storage_arr.data());
    const size_t n_storage = (size_t)storage_arr.size();
    int rc;
    {
      py::gil_scoped_release release;
      rc = hctr_create(&cfg, root, storage, n_storage, &table_);
    }
    if (rc) raise_last();
  }
  TableContainer(const TableContainer &) = delete;
  TableContainer &operator=(const TableContainer &) = delete;
  ~TableContainer() {
    pool_.reset(); // runs what is still queued, then joins
    if (table_) hctr_destroy(table_);
  }

  void pushPull(unsigned long grad, unsigned long dst) {
    py::gil_scoped_release release;
    if (hctr_push_pull(table_, reinterpret_cast<const float *>(grad), reinterpret_cast<float *>(dst))) raise_last();
  }
  void preprocess(unsigned long data_ptr, size_t batch_size) {
    py::gil_scoped_release release;
    if (hctr_preprocess(table_, reinterpret_cast<const int64_t *>(data_ptr), batch_size)) raise_last();
  }
  std::shared_future<void> pushPullAsync(unsigned long grad, unsigned long dst) {
    if (!pool_) pool_ = std::make_unique<SerialWorker>();
    hctr_table *t = table_;
    return pool_->enqueue([t, grad, dst] {
      if (hctr_push_pull(t, reinterpret_cast<const float *>(grad), reinterpret_cast<float *>(dst))) raise_last();
    });
  }
  std::shared_future<void> preprocessAsync(unsigned long data_ptr, size_t batch_size) {
    if (!pool_) pool_ = std::make_unique<SerialWorker>();
    hctr_table *t = table_;
    return pool_->enqueue([t, data_ptr, batch_size] {
      if (hctr_preprocess(t, reinterpret_cast<const int64_t *>(data_ptr), batch_size)) raise_last();
    });
  }
  std::string debugString() {
    char b[256];
    hctr_repr(table_, b, sizeof b);
    return b;
  }
  std::string debugStringFull() {
    char b[512];
    hctr_debug(table_, b, sizeof b);
    return b;
  }
  // additive: integer intermediates and table state as numpy arrays (HCTR_F_* item numbers)
  py::array debugFetch(int which) {
    size_t n = 0;
    if (hctr_debug_fetch(table_, which, nullptr, 0, &n)) raise_last();
    if (which == HCTR_F_EMBEDDING || which == HCTR_F_PENDING) {
      py::array_t<float> out(n);
      if (hctr_debug_fetch(table_, which, out.mutable_data(), n, &n)) raise_last();
      return std::move(out);
    }
    py::array_t<long long> out(n);
    if (hctr_debug_fetch(table_, which, out.mutable_data(), n, &n)) raise_last();
    return std::move(out);
  }
  void callTiming(bool on) {
    if (hctr_call_timing(table_, on ? 1 : 0)) raise_last();
  }
  py::tuple lastTimes() {
    float a = 0, b = 0;
    if (hctr_last_times(table_, &a, &b)) raise_last();
    return py::make_tuple(a, b);
  }

 private:
  hctr_table *table_ = nullptr;
  std::unique_ptr<SerialWorker> pool_;
};

} // namespace

PYBIND11_MODULE(hetuCTR, m) {
  m.doc() = "hetuCTR embedding table, HIP implementation for MI355X (gfx950)";

  typedef std::shared_future<void> wait_t;
  py::class_<wait_t>(m, "_waittype").def("wait", [](const wait_t &w) {
    py::gil_scoped_release release;
    w.get(); // rethrows what the call raised on the worker thread
  });

  py::enum_<InitType>(m, "InitType", py::module_local())
      .value("Zero", InitType::kZero)
      .value("Normal", InitType::kNormal)
      .value("TruncatedNormal", InitType::kTruncatedNormal)
      .value("Uniform", InitType::kUniform);

  py::class_<Initializer>(m, "Initializer", py::module_local()).def(py::init<InitType, float, float>());

  py::class_<TableContainer>(m, "HetuTable", py::module_local())
      .def(py::init<int, int, int, const std::string &, int, size_t, size_t, long long, long long, py::array_t<uint8_t>,
                    py::array_t<long long>, const Initializer &, float, int>(),
           py::arg("rank"), py::arg("nrank"), py::arg("device_id"), py::arg("ip"), py::arg("port"), py::arg("length"),
           py::arg("width"), py::arg("pull_bound"), py::arg("push_bound"), py::arg("root_arr"), py::arg("storage_arr"),
           py::arg("init"), py::arg("learning_rate"), py::arg("verbose"))
      .def("preprocess", &TableContainer::preprocess)
      .def("push_pull", &TableContainer::pushPull)
      .def("async_push_pull", &TableContainer::pushPullAsync)
      .def("async_preprocess", &TableContainer::preprocessAsync)
      .def("__repr__", &TableContainer::debugString)
      .def("debug", &TableContainer::debugStringFull)
      .def("debug_fetch", &TableContainer::debugFetch, py::arg("which"))
      .def("call_timing", &TableContainer::callTiming, py::arg("on"))
      .def("last_times", &TableContainer::lastTimes);

  m.def("seed", [](unsigned long seed) { hctr_seed(seed); });
  m.def("version", [] { return std::string(hctr_version()); });
  m.def("last_error", [] { return std::string(hctr_last_error()); });
}
