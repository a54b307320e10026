// Small host-side helpers of the model layer: error check that throws (the
// reference's CHECK_GPU_ERROR, lightseq/inference/tools/util.h:69-79), a device
// buffer owner and host<->device copies.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <stdexcept>
#include <string>
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

inline std::vector<__half> to_half(const std::vector<float>& v) {
  std::vector<__half> out(v.size());
  for (size_t i = 0; i < v.size(); ++i) out[i] = __float2half_rn(v[i]);
  return out;
}

}  // namespace hip
}  // namespace lightseq
