// Process-wide launch context of the layer API: the stream every layer launches on
// (the reference's Context singleton, lightseq/csrc/ops/includes/context.h:14-43, without
// its cuBLAS handles -- the GEMMs here are this library's own kernels).
#pragma once

#include <hip/hip_runtime.h>

namespace lightseq {
namespace hip {

class Context {
 public:
  static Context& Instance() {
    static Context ctx;
    return ctx;
  }
  void set_stream(hipStream_t stream) { _stream = stream; }
  hipStream_t get_stream() const { return _stream; }

 private:
  Context() : _stream(nullptr) {}
  hipStream_t _stream;
};

}  // namespace hip
}  // namespace lightseq
