// lightseq/csrc/layers/quant_linear_layer.cpp:7-60, int8 branch: quantise the input and the
// weight, int8 GEMM to int8 with alpha = c_in * c_w / (c_out * 127) read from device
// memory, dequantise with the output clip.
#include "quant_linear_layer.h"

#include "context.h"

namespace lightseq {
namespace hip {

using namespace lsh;

template <typename T>
QuantLinearLayer<T>::QuantLinearLayer(int layer_id, int in_features, int out_features,
                                      int max_batch_tokens)
    : _layer_id(layer_id),
      _in_features(in_features),
      _out_features(out_features),
      _max_batch_tokens(max_batch_tokens) {
  if (in_features <= 0 || out_features <= 0 || max_batch_tokens <= 0)
    throw std::runtime_error("QuantLinearLayer: sizes must be positive");
  if (in_features % 16 != 0)
    throw std::runtime_error("QuantLinearLayer: in_features must be a multiple of 16");
  _quant_input.alloc((size_t)max_batch_tokens * in_features);
  _quant_weight.alloc((size_t)in_features * out_features);
  _quant_output.alloc((size_t)max_batch_tokens * out_features);
  _igemm_alpha.alloc(max_batch_tokens);
}

template <typename T>
void QuantLinearLayer<T>::set_cur_batch_shape(int batch_size, int seq_len) {
  if (batch_size <= 0 || seq_len <= 0 || (long)batch_size * seq_len > _max_batch_tokens)
    throw std::runtime_error("QuantLinearLayer: batch tokens exceed max_batch_tokens");
  _batch_size = batch_size;
  _seq_len = seq_len;
}

template <typename T>
void QuantLinearLayer<T>::SetQuantMode(bool enable_quant) { _enable_quant = enable_quant; }

template <typename T>
void QuantLinearLayer<T>::Forward(const T* inputs_ptr, const T* weight_ptr, const T* cmax_ptr,
                                  T* outputs_ptr) {
  if (!inputs_ptr || !weight_ptr || !cmax_ptr || !outputs_ptr)
    throw std::runtime_error("QuantLinearLayer::Forward: null pointer");
  if (!_enable_quant)
    throw std::runtime_error(
        "QuantLinearLayer::Forward: only the quantised path of the layer is provided");
  const int tok = _batch_size * _seq_len;
  if (tok == 0) throw std::runtime_error("QuantLinearLayer::Forward: set_cur_batch_shape not called");
  hipStream_t stream = Context::Instance().get_stream();
  LSH_CALL(opb_quantize<T>(_quant_input.get(), nullptr, _igemm_alpha.get(), inputs_ptr, cmax_ptr,
                           (long)tok * _in_features, 1, 2, stream));
  LSH_CALL(opb_quantize<T>(_quant_weight.get(), nullptr, nullptr, weight_ptr, cmax_ptr + 1,
                           (long)_in_features * _out_features, 0, 4, stream));
  LSH_CALL(gemm_i8_i8o_dev_alpha(_quant_input.get(), _quant_weight.get(), _quant_output.get(), tok,
                                 _out_features, _in_features, _igemm_alpha.get(), stream));
  LSH_CALL(opb_dequantize<T>(outputs_ptr, _quant_output.get(), cmax_ptr + 2,
                             (long)tok * _out_features, stream));
}

template class QuantLinearLayer<__half>;

}  // namespace hip
}  // namespace lightseq
