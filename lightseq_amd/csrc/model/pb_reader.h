// Minimal protobuf wire-format reader: enough for LightSeq's quantised model files
// (varint, 32/64-bit and length-delimited fields; packed or unpacked repeated
// floats).  No schema compiler and no protobuf runtime are involved.
#pragma once

#include <stdint.h>
#include <string.h>

#include <stdexcept>
#include <string>
#include <vector>

namespace lsh {

struct PbField {
  int number = 0;
  int wire = 0;             // 0 varint, 1 fixed64, 2 length-delimited, 5 fixed32
  uint64_t varint = 0;      // wire 0
  const uint8_t* data = 0;  // wire 1, 2, 5
  size_t size = 0;

  float as_float() const {
    if (wire != 5) throw std::runtime_error("protobuf: field is not a 32-bit float");
    float f;
    memcpy(&f, data, 4);
    return f;
  }
  int32_t as_int32() const {
    if (wire != 0) throw std::runtime_error("protobuf: field is not a varint");
    return (int32_t)(int64_t)varint;
  }
  bool as_bool() const { return as_int32() != 0; }
  std::string as_string() const {
    if (wire != 2) throw std::runtime_error("protobuf: field is not length-delimited");
    return std::string(reinterpret_cast<const char*>(data), size);
  }
  // appends the floats of a packed (wire 2) or single unpacked (wire 5) repeated field
  void append_floats(std::vector<float>& out) const {
    if (wire == 5) {
      out.push_back(as_float());
    } else if (wire == 2) {
      if (size % 4) throw std::runtime_error("protobuf: packed float field of odd size");
      size_t n = size / 4, old = out.size();
      out.resize(old + n);
      memcpy(out.data() + old, data, size);
    } else {
      throw std::runtime_error("protobuf: field is not a repeated float");
    }
  }
};

class PbReader {
 public:
  PbReader(const uint8_t* p, size_t n) : p_(p), end_(p + n) {}
  explicit PbReader(const PbField& f) : p_(f.data), end_(f.data + f.size) {
    if (f.wire != 2) throw std::runtime_error("protobuf: embedded message expected");
  }

  // Reads the next field; false at the end of the message.
  bool next(PbField& f) {
    if (p_ >= end_) return false;
    uint64_t key = varint();
    f.number = (int)(key >> 3);
    f.wire = (int)(key & 7);
    f.data = nullptr;
    f.size = 0;
    switch (f.wire) {
      case 0: f.varint = varint(); break;
      case 1: take(f, 8); break;
      case 5: take(f, 4); break;
      case 2: {
        uint64_t n = varint();
        if (n > (uint64_t)(end_ - p_)) throw std::runtime_error("protobuf: truncated field");
        take(f, (size_t)n);
        break;
      }
      default: throw std::runtime_error("protobuf: unsupported wire type");
    }
    return true;
  }

 private:
  uint64_t varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 64; shift += 7) {
      if (p_ >= end_) throw std::runtime_error("protobuf: truncated varint");
      uint8_t b = *p_++;
      v |= (uint64_t)(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    throw std::runtime_error("protobuf: varint too long");
  }
  void take(PbField& f, size_t n) {
    if (n > (size_t)(end_ - p_)) throw std::runtime_error("protobuf: truncated field");
    f.data = p_;
    f.size = n;
    p_ += n;
  }
  const uint8_t* p_;
  const uint8_t* end_;
};

}  // namespace lsh
