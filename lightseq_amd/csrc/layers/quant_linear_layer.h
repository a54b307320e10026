// Quantised linear layer behind the reference's interface
// (lightseq/csrc/layers/includes/quant_linear_layer.h:14-33).  Forward only, fp16.
#pragma once

#include "../model/model_util.h"

namespace lightseq {
namespace hip {

template <typename T>
class QuantLinearLayer {
 public:
  QuantLinearLayer(int layer_id, int in_features, int out_features, int max_batch_tokens);
  // cmax_ptr: three device scalars (input, weight, output clip)
  void Forward(const T* inputs_ptr, const T* weight_ptr, const T* cmax_ptr, T* outputs_ptr);
  void set_cur_batch_shape(int batch_size, int seq_len);
  void SetQuantMode(bool enable_quant);

 private:
  const int _layer_id, _in_features, _out_features, _max_batch_tokens;
  bool _enable_quant = false;
  int _batch_size = 0, _seq_len = 0;
  DeviceBuffer<int8_t> _quant_input, _quant_weight, _quant_output;
  DeviceBuffer<float> _igemm_alpha;
};

}  // namespace hip
}  // namespace lightseq
