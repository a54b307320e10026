// C++ model interface of the library: the same abstract class, factory and
// registration macro as the reference's lightseq::cuda::LSModel
// (lightseq/inference/pywrapper/model_base.h:12-148), in namespace lightseq::hip.
// Errors are C++ exceptions (std::runtime_error), as in the reference; the C ABI in
// include/lightseq_model.h turns them into status codes.
#pragma once

#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace lightseq {
namespace hip {

enum DataType {
  kNotSupported = 0, kFloat32 = 1, kInt32 = 2, kInt64 = 3, kFloat16 = 4, kInt8 = 5, kInt16 = 6,
  kByte = 7, kUInt8 = 8, kUInt16 = 9, kUInt32 = 10, kUInt64 = 11, kFloat64 = 12
};

// One input or output of a model: what the accessor functions of LSModel answer from.  `slot`
// is where the model keeps the device pointer of this tensor (inside its encoder / decoder).
struct IoSlot {
  DataType dtype = kNotSupported;
  std::vector<int> max_shape;
  void** slot = nullptr;
};

class LSModel {
 public:
  LSModel(std::vector<std::string> input_names, std::vector<std::string> output_names)
      : kInputNames(std::move(input_names)), kOutputNames(std::move(output_names)) {
    input_shapes_.resize(kInputNames.size());
    output_shapes_.resize(kOutputNames.size());
    inputs_.resize(kInputNames.size());
    outputs_.resize(kOutputNames.size());
  }
  virtual ~LSModel() {}
  virtual void Infer() = 0;

  // The accessors below are answered from the descriptor table that the model's constructor
  // fills (describe_input / describe_output); a model overrides none of them.
  virtual void set_input_ptr(int index, void* input_ptr) { *slot_of(inputs_, index, "input").slot = input_ptr; }
  void set_input_shape(int index, std::vector<int> shape) {
    input_shapes_.at(index) = std::move(shape);
  }
  virtual std::vector<int> get_input_max_shape(int index) {
    return slot_of(inputs_, index, "input").max_shape;
  }
  std::string get_input_name(int index) { return kInputNames.at(index); }
  int get_input_size() { return (int)kInputNames.size(); }
  virtual DataType get_input_dtype(int index) { return slot_of(inputs_, index, "input").dtype; }

  virtual void set_output_ptr(int index, void* output_ptr) {
    *slot_of(outputs_, index, "output").slot = output_ptr;
  }
  virtual const void* get_output_ptr(int index) { return *slot_of(outputs_, index, "output").slot; }
  std::string get_output_name(int index) { return kOutputNames.at(index); }
  int get_output_size() { return (int)kOutputNames.size(); }
  std::vector<int> get_output_shape(int index) { return output_shapes_.at(index); }
  virtual std::vector<int> get_output_max_shape(int index) {
    return slot_of(outputs_, index, "output").max_shape;
  }
  virtual DataType get_output_dtype(int index) { return slot_of(outputs_, index, "output").dtype; }

  virtual void benchmark_mode(bool is_benchmark) = 0;

  // Not in the reference: the HIP stream the model launches on (for event timing).
  virtual void* get_stream() = 0;

 protected:
  void set_output_shape(int index, std::vector<int> shape) {
    output_shapes_.at(index) = std::move(shape);
  }
  template <typename T>
  void describe_input(int index, DataType dtype, std::vector<int> max_shape, T** slot) {
    inputs_.at(index) = IoSlot{dtype, std::move(max_shape), (void**)slot};
  }
  template <typename T>
  void describe_output(int index, DataType dtype, std::vector<int> max_shape, T** slot) {
    outputs_.at(index) = IoSlot{dtype, std::move(max_shape), (void**)slot};
  }
  const std::vector<std::string> kInputNames;
  const std::vector<std::string> kOutputNames;
  std::vector<std::vector<int>> input_shapes_;
  std::vector<std::vector<int>> output_shapes_;

 private:
  static IoSlot& slot_of(std::vector<IoSlot>& table, int index, const char* what) {
    if (index < 0 || index >= (int)table.size() || table[index].slot == nullptr)
      throw std::runtime_error(std::string("invalid ") + what + " index");
    return table[index];
  }
  std::vector<IoSlot> inputs_, outputs_;
};

typedef LSModel* (*LSModelConstructor)(const std::string, const int);

class LSModelFactory {
 public:
  static LSModelFactory& GetInstance() {
    static LSModelFactory factory;
    return factory;
  }
  void ModelRegister(std::string class_name, LSModelConstructor obj) {
    if (obj) object_map_.insert({class_name, obj});
  }
  LSModel* CreateModel(std::string class_name, const std::string weight_path,
                       const int max_batch_size) {
    auto iter = object_map_.find(class_name);
    if (iter == object_map_.end()) throw std::runtime_error("Model not supported");
    return iter->second(weight_path, max_batch_size);
  }

 private:
  LSModelFactory() {}
  std::map<std::string, LSModelConstructor> object_map_;
};

class Reflector {
 public:
  Reflector(std::string name, LSModelConstructor obj) {
    LSModelFactory::GetInstance().ModelRegister(name, obj);
  }
};

#define LSMODEL_REGISTER(className)                                                         \
  LSModel* create_object_##className(const std::string weight_path,                         \
                                     const int max_batch_size) {                            \
    return new className(weight_path, max_batch_size);                                      \
  }                                                                                         \
  Reflector reflector_##className(#className, create_object_##className);

}  // namespace hip
}  // namespace lightseq
