// Small host-side helpers of the model layer: error check that throws (the
// reference's CHECK_GPU_ERROR, lightseq/inference/tools/util.h:69-79), a device
// buffer owner and host<->device copies.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <list>
#include <map>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "../ls_launch.h"

namespace lightseq {
namespace hip {

inline void check_gpu_error(hipError_t e, const char* file, int line) {
  if (e != hipSuccess)
    throw std::runtime_error(std::string("[HIP][ERROR] ") + file + "(" + std::to_string(line) +
                             "): " + hipGetErrorName(e) + " " + hipGetErrorString(e));
}
#define CHECK_GPU_ERROR(val) ::lightseq::hip::check_gpu_error((val), __FILE__, __LINE__)

// status of a library launcher -> exception carrying its message
inline void check_status(int rc) {
  if (rc != LSH_OK) throw std::runtime_error(lsh_last_error());
}
#define LSH_CALL(expr) ::lightseq::hip::check_status((expr))

// Owning device allocation.
template <typename T>
class DeviceBuffer {
 public:
  DeviceBuffer() {}
  explicit DeviceBuffer(size_t n) { alloc(n); }
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  DeviceBuffer(DeviceBuffer&& o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
  DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
    if (this != &o) { release(); p_ = o.p_; n_ = o.n_; o.p_ = nullptr; o.n_ = 0; }
    return *this;
  }
  ~DeviceBuffer() { release(); }
  void alloc(size_t n) {
    release();
    if (n == 0) return;
    CHECK_GPU_ERROR(hipMalloc(reinterpret_cast<void**>(&p_), n * sizeof(T)));
    n_ = n;
  }
  void upload(const T* host, size_t n, hipStream_t s) {
    if (n > n_) throw std::runtime_error("DeviceBuffer::upload: too large");
    CHECK_GPU_ERROR(hipMemcpyAsync(p_, host, n * sizeof(T), hipMemcpyHostToDevice, s));
  }
  T* get() const { return p_; }
  size_t size() const { return n_; }

 private:
  void release() {
    if (p_) (void)hipFree(p_);
    p_ = nullptr;
    n_ = 0;
  }
  T* p_ = nullptr;
  size_t n_ = 0;
};

// A HIP stream of the default priority that is destroyed with its owner.
class StreamOwner {
 public:
  StreamOwner() = default;
  StreamOwner(const StreamOwner&) = delete;
  StreamOwner& operator=(const StreamOwner&) = delete;
  ~StreamOwner() {
    if (s_) (void)hipStreamDestroy(s_);
  }
  void create() {
    if (!s_) CHECK_GPU_ERROR(hipStreamCreate(&s_));
  }
  hipStream_t get() const { return s_; }
  operator hipStream_t() const { return s_; }

 private:
  hipStream_t s_ = nullptr;
};

// Three HIP events on the model's stream per Infer() of a generation model: entry, start of the
// step loop, end of the step loop.  times() is valid once the stream has been synchronised.
class PhaseEvents {
 public:
  PhaseEvents() = default;
  PhaseEvents(const PhaseEvents&) = delete;
  PhaseEvents& operator=(const PhaseEvents&) = delete;
  ~PhaseEvents() {
    for (hipEvent_t e : ev_)
      if (e) (void)hipEventDestroy(e);
  }
  void mark(int i, hipStream_t s) {
    if (!ev_[i]) CHECK_GPU_ERROR(hipEventCreate(&ev_[i]));
    CHECK_GPU_ERROR(hipEventRecord(ev_[i], s));
    if (i == 0) loop_steps_ = 0;
    marked_ |= 1 << i;
  }
  void set_loop_steps(int n) { loop_steps_ = n; }
  // milliseconds before the step loop and inside it, steps the loop ran; false before a run
  bool times(float* prepare_ms, float* steps_ms, int* steps) const {
    if (marked_ != 7) return false;
    CHECK_GPU_ERROR(hipEventElapsedTime(prepare_ms, ev_[0], ev_[1]));
    CHECK_GPU_ERROR(hipEventElapsedTime(steps_ms, ev_[1], ev_[2]));
    *steps = loop_steps_;
    return true;
  }

 private:
  hipEvent_t ev_[3] = {nullptr, nullptr, nullptr};
  int marked_ = 0, loop_steps_ = 0;
};

// Debug taps of a generation step (parity bisection): device-to-device copies of named
// intermediates of decoder layer `layer` at step `step` into buffers the caller owns.  A name
// registered with a null pointer is forgotten.  A layer < 0 at the copy site means "any".
class StepTaps {
 public:
  void set(int layer, const std::string& name, void* dst) {
    _layer = layer;
    if (dst) _dst[name] = dst;
    else _dst.erase(name);
  }
  void set_step(int step) { _step = step; }
  bool any() const { return !_dst.empty(); }
  bool wants(int layer, int step, const char* name) const {
    return !_dst.empty() && step == _step && (layer < 0 || layer == _layer) && _dst.count(name);
  }
  void copy(int layer, int step, const char* name, const void* src, size_t bytes,
            hipStream_t stream) const {
    if (!wants(layer, step, name)) return;
    if (hipMemcpyAsync(_dst.at(name), src, bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess)
      throw std::runtime_error(std::string("tap copy failed: ") + name);
  }

 private:
  int _layer = -1, _step = -1;
  std::map<std::string, void*> _dst;
};

// HIP graphs of a generation step.  A step is a fixed sequence of launches whose arguments
// depend only on the shapes of the call and on the position of the step, so the sequence
// enqueued for one key is the sequence for every later call with that key -- as long as the
// process-wide route switches stand as they stood at the capture (route_epoch(); a change drops
// every graph held) and the body bakes in no pointer that a caller can replace.
//   first time a key is seen   the step runs eagerly (kernel attributes get set, nothing is kept)
//   second time                the step is captured from the stream, instantiated and launched
//   later                      one hipGraphLaunch
// At most kMaxGraphs executables are kept, the least recently launched one is destroyed first.
// A key whose capture or instantiation fails runs eagerly from then on.
// The body may only enqueue kernels and device-to-device copies on the stream: no memset nodes
// (they replay wrongly on this platform), no synchronisation, no host reads.
class StepGraphs {
 public:
  StepGraphs() {}
  StepGraphs(const StepGraphs&) = delete;
  StepGraphs& operator=(const StepGraphs&) = delete;
  ~StepGraphs() { clear(); }
  void clear() {
    for (auto& kv : execs_) (void)hipGraphExecDestroy(kv.second.exec);
    execs_.clear();
    lru_.clear();
    seen_.clear();
    eager_only_.clear();
  }
  int captured() const { return captured_; }
  long replayed() const { return replayed_; }
  size_t held() const { return execs_.size(); }
  int last_graph_nodes() const { return last_nodes_; }  // launches of the step captured last
  static constexpr size_t kMaxGraphs = 512;

  template <typename Body>
  void run(uint64_t key, hipStream_t stream, bool enabled, Body&& body) {
    if (!enabled) {
      body();
      return;
    }
    const unsigned long epoch = lsh::route_epoch();
    if (epoch != epoch_) {
      clear();
      epoch_ = epoch;
    }
    auto it = execs_.find(key);
    if (it != execs_.end()) {
      lru_.splice(lru_.begin(), lru_, it->second.pos);
      CHECK_GPU_ERROR(hipGraphLaunch(it->second.exec, stream));
      ++replayed_;
      return;
    }
    if (eager_only_.count(key) || seen_.insert(key).second) {  // failed before / first encounter
      body();
      return;
    }
    hipGraphExec_t exec = capture(stream, body);
    if (!exec) {  // the platform refused: the step still has to run
      eager_only_.insert(key);
      body();
      return;
    }
    while (execs_.size() >= kMaxGraphs) {
      const uint64_t old = lru_.back();
      lru_.pop_back();
      auto o = execs_.find(old);
      (void)hipGraphExecDestroy(o->second.exec);
      execs_.erase(o);
    }
    lru_.push_front(key);
    execs_[key] = Held{exec, lru_.begin()};
    ++captured_;
    CHECK_GPU_ERROR(hipGraphLaunch(exec, stream));
    ++replayed_;
  }

 private:
  struct Held {
    hipGraphExec_t exec;
    std::list<uint64_t>::iterator pos;
  };
  // Records the body; null when the capture or the instantiation fails (nothing has run then).
  // An exception of the body itself (a launcher that rejects its arguments) propagates.
  template <typename Body>
  hipGraphExec_t capture(hipStream_t stream, Body&& body) {
    if (hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    hipGraph_t graph = nullptr;
    try {
      body();
    } catch (...) {
      (void)hipStreamEndCapture(stream, &graph);
      if (graph) (void)hipGraphDestroy(graph);
      throw;
    }
    if (hipStreamEndCapture(stream, &graph) != hipSuccess || !graph) {
      (void)hipGetLastError();
      if (graph) (void)hipGraphDestroy(graph);
      return nullptr;
    }
    size_t nodes = 0;
    if (hipGraphGetNodes(graph, nullptr, &nodes) == hipSuccess) last_nodes_ = (int)nodes;
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    return exec;
  }
  std::unordered_map<uint64_t, Held> execs_;
  std::list<uint64_t> lru_;  // most recently launched first
  std::unordered_set<uint64_t> seen_, eager_only_;
  unsigned long epoch_ = 0;
  int captured_ = 0, last_nodes_ = 0;
  long replayed_ = 0;
};

inline std::vector<__half> to_half(const std::vector<float>& v) {
  std::vector<__half> out(v.size());
  for (size_t i = 0; i < v.size(); ++i) out[i] = __float2half_rn(v[i]);
  return out;
}

// float vector -> fp16 on the device
inline DeviceBuffer<__half> upload_half(const std::vector<float>& v, hipStream_t s) {
  std::vector<__half> h = to_half(v);
  DeviceBuffer<__half> d(h.size());
  d.upload(h.data(), h.size(), s);
  CHECK_GPU_ERROR(hipStreamSynchronize(s));  // `h` dies at return
  return d;
}

// stored uint8 [rows(in), cols(out)] -> int8 [cols, rows] (K-contiguous for the GEMM)
inline DeviceBuffer<int8_t> upload_kernel(const std::vector<uint8_t>& w, int rows, int cols,
                                          bool transpose, hipStream_t s) {
  DeviceBuffer<uint8_t> raw(w.size());
  raw.upload(w.data(), w.size(), s);
  DeviceBuffer<int8_t> q(w.size());
  LSH_CALL(lsh::stored_u8_to_i8(raw.get(), q.get(), rows, cols, transpose, s));
  CHECK_GPU_ERROR(hipStreamSynchronize(s));
  return q;
}

}  // namespace hip
}  // namespace lightseq
