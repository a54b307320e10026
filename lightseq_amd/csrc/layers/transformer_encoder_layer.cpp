// Forward pass of the quantised encoder layer
// (lightseq/csrc/layers/transformer_encoder_layer.cpp:66-293), built from this library's
// operator kernels.  What differs from the reference's sequence is only where kernels are
// fused: the attention core (scores, masked softmax, context, head merge) is one kernel,
// and the int8 GEMMs read their scale from device memory in the epilogue.
#include "transformer_encoder_layer.h"

#include <algorithm>

#include "context.h"

namespace lightseq {
namespace hip {

using namespace lsh;

template <typename T>
TransformerEncoderLayer<T>::TransformerEncoderLayer(
    int layer_id, int max_batch_tokens, int max_seq_len, int hidden_size, int num_heads,
    int intermediate_size, float attn_prob_dropout_ratio, float activation_dropout_ratio,
    float hidden_output_dropout_ratio, bool pre_or_postLayerNorm, std::string activation_fn,
    bool mask_future_tokens)
    : _layer_id(layer_id),
      _max_batch_tokens(max_batch_tokens),
      _max_seq_len(max_seq_len),
      _hidden_size(hidden_size),
      _heads(num_heads),
      _intermediate_size(intermediate_size),
      _is_pre_ln(pre_or_postLayerNorm),
      _activation_fn(activation_fn),
      _mask_future_tokens(mask_future_tokens) {
  (void)attn_prob_dropout_ratio;  // ratios only matter in training mode, which Forward rejects
  (void)activation_dropout_ratio;
  (void)hidden_output_dropout_ratio;
  if (max_batch_tokens <= 0 || max_seq_len <= 0 || hidden_size <= 0 || num_heads <= 0 ||
      intermediate_size <= 0)
    throw std::runtime_error("TransformerEncoderLayer: sizes must be positive");
  if (hidden_size % num_heads != 0)
    throw std::runtime_error("TransformerEncoderLayer: hidden_size % num_heads != 0");
  const int hd = hidden_size / num_heads;
  if (hd != 32 && hd != 64 && hd != 128)
    throw std::runtime_error("TransformerEncoderLayer: head dim must be 32, 64 or 128");
  if (hidden_size % 16 != 0 || intermediate_size % 16 != 0)
    throw std::runtime_error(
        "TransformerEncoderLayer: hidden and intermediate size must be multiples of 16");
  if (activation_fn != "relu" && activation_fn != "gelu")
    throw std::runtime_error("not supported activation: " + activation_fn);

  const size_t tok = (size_t)max_batch_tokens, hs = (size_t)hidden_size,
               ims = (size_t)intermediate_size;
  if (_is_pre_ln) _ln_out.alloc(tok * hs);
  _qkv.alloc(3 * tok * hs);
  _attn_o_inp.alloc(tok * hs);
  _ffn_inp.alloc(tok * hs);
  _ff2_inp.alloc(tok * ims);
  _fake_weight.alloc(hs * ims);
  _vars.alloc(tok);
  _qin.alloc(tok * std::max(hs, ims));
  _qout.alloc(tok * std::max(3 * hs, ims));
  _qweight.alloc(std::max(3 * hs * hs, hs * ims));
  _igemm_alpha.alloc(tok);
}

template <typename T>
size_t TransformerEncoderLayer<T>::param_count() const {
  const size_t hs = _hidden_size, ims = _intermediate_size;
  return hs * hs * 3 + hs * 3 + hs * hs + hs + hs + hs + hs * ims + ims + hs * ims + hs + hs +
         hs + 12;
}

template <typename T>
void TransformerEncoderLayer<T>::assign_weight_ptr(const T* weights_ptr) {
  if (!weights_ptr) throw std::runtime_error("assign_weight_ptr: null parameter blob");
  const size_t hs = _hidden_size, ims = _intermediate_size;
  const T* wptr = weights_ptr;
  _attn_qkvw_ptr = wptr; wptr += hs * hs * 3;
  _attn_qkvb_ptr = wptr; wptr += hs * 3;
  _attn_ow_ptr = wptr;   wptr += hs * hs;
  _attn_ob_ptr = wptr;   wptr += hs;
  _attn_nw_ptr = wptr;   wptr += hs;
  _attn_nb_ptr = wptr;   wptr += hs;
  _inter_w_ptr = wptr;   wptr += hs * ims;
  _inter_b_ptr = wptr;   wptr += ims;
  _output_w_ptr = wptr;  wptr += hs * ims;
  _output_b_ptr = wptr;  wptr += hs;
  _ffn_nw_ptr = wptr;    wptr += hs;
  _ffn_nb_ptr = wptr;    wptr += hs;
  _attn_qkv_cmax_ptr = wptr;       wptr += 3;
  _attn_out_cmax_ptr = wptr;       wptr += 3;
  _inter_cmax_ptr = wptr;          wptr += 3;
  _output_cmax_ptr = wptr;         wptr += 2;
  _attn_qkv_cache_cmax_ptr = wptr; wptr += 1;
}

template <typename T>
void TransformerEncoderLayer<T>::set_cur_batch_shape(int batch_size, int seq_len) {
  if (batch_size <= 0 || seq_len <= 0)
    throw std::runtime_error("set_cur_batch_shape: batch_size and seq_len must be positive");
  if ((long)batch_size * seq_len > _max_batch_tokens)
    throw std::runtime_error("Batch token numbers " + std::to_string((long)batch_size * seq_len) +
                             " exceeds the limit " + std::to_string(_max_batch_tokens) + ".");
  if (seq_len > _max_seq_len)
    throw std::runtime_error("Sequence length " + std::to_string(seq_len) +
                             " exceeds the limit " + std::to_string(_max_seq_len) + ".");
  _batch_size = batch_size;
  _seq_len = seq_len;
  _batch_tokens = batch_size * seq_len;
}

template <typename T>
void TransformerEncoderLayer<T>::SetTrainingMode(bool training) { _training = training; }

template <typename T>
void TransformerEncoderLayer<T>::SetQuantMode(bool enable_quant) { _enable_quant = enable_quant; }

// transformer_encoder_layer.cpp:66-185
template <typename T>
void TransformerEncoderLayer<T>::attn_layer_fw(const T* input_ptr, const T* input_mask_ptr,
                                               T* output_ptr) {
  const int tok = _batch_tokens, hs = _hidden_size;
  if (_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(_ln_out.get(), nullptr, nullptr, _vars.get(), nullptr, input_ptr,
                               _attn_nw_ptr, _attn_nb_ptr, nullptr, tok, hs, _stream));
  const T* gemmQKV_inp_ptr = _is_pre_ln ? _ln_out.get() : input_ptr;

  LSH_CALL(opb_quantize<T>(_qin.get(), nullptr, _igemm_alpha.get(), gemmQKV_inp_ptr,
                           _attn_qkv_cmax_ptr, (long)tok * hs, tok, 2, _stream));
  LSH_CALL(opb_quantize<T>(_qweight.get(), nullptr, nullptr, _attn_qkvw_ptr,
                           _attn_qkv_cmax_ptr + 1, 3L * hs * hs, 0, 4, _stream));
  LSH_CALL(gemm_i8_i8o_dev_alpha(_qin.get(), _qweight.get(), _qout.get(), tok, 3 * hs, hs,
                                 _igemm_alpha.get(), _stream));
  const T* cache_cmax = _mask_future_tokens ? _attn_qkv_cache_cmax_ptr : nullptr;
  LSH_CALL(opb_quant_bias_add_transform_20314<T>(_qkv.get(), nullptr, _qout.get(), _attn_qkvb_ptr,
                                                 _attn_qkv_cmax_ptr + 2, _batch_size, _seq_len, 3,
                                                 _heads, hs / _heads, _stream, cache_cmax));

  // scores, masked softmax, context and head merge in one kernel (:121-148)
  const size_t batch_dim = (size_t)tok * hs;
  const T* q = _qkv.get();
  LSH_CALL(layer_attention_f16(q, q + batch_dim, q + 2 * batch_dim, input_mask_ptr,
                               _attn_o_inp.get(), _batch_size, _seq_len, _heads, hs / _heads,
                               _mask_future_tokens, _stream));

  LSH_CALL(opb_quantize<T>(_qin.get(), nullptr, _igemm_alpha.get(), _attn_o_inp.get(),
                           _attn_out_cmax_ptr, (long)tok * hs, tok, 2, _stream));
  LSH_CALL(opb_quantize<T>(_qweight.get(), nullptr, nullptr, _attn_ow_ptr, _attn_out_cmax_ptr + 1,
                           (long)hs * hs, 0, 4, _stream));
  LSH_CALL(gemm_i8_i8o_dev_alpha(_qin.get(), _qweight.get(), _qout.get(), tok, hs, hs,
                                 _igemm_alpha.get(), _stream));
  LSH_CALL(opb_quant_dropout_res_bias<T>(output_ptr, nullptr, _qout.get(), _attn_out_cmax_ptr + 2,
                                         _attn_ob_ptr, input_ptr, (long)tok * hs, hs, 0.f,
                                         _stream));
  if (!_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(output_ptr, nullptr, nullptr, _vars.get(), nullptr, output_ptr,
                               _attn_nw_ptr, _attn_nb_ptr, nullptr, tok, hs, _stream));
}

// transformer_encoder_layer.cpp:188-250
template <typename T>
void TransformerEncoderLayer<T>::ffn_layer_fw(T* inp_ptr, T* out_ptr) {
  const int tok = _batch_tokens, hs = _hidden_size, ims = _intermediate_size;
  const T* ff1_inp = inp_ptr;
  if (_is_pre_ln) {
    LSH_CALL(opb_layer_norm<T>(_ln_out.get(), nullptr, nullptr, _vars.get(), nullptr, inp_ptr,
                               _ffn_nw_ptr, _ffn_nb_ptr, nullptr, tok, hs, _stream));
    ff1_inp = _ln_out.get();
  }
  LSH_CALL(opb_quantize<T>(_qin.get(), nullptr, _igemm_alpha.get(), ff1_inp, _inter_cmax_ptr,
                           (long)tok * hs, tok, 2, _stream));
  LSH_CALL(opb_quantize<T>(_qweight.get(), nullptr, nullptr, _inter_w_ptr, _inter_cmax_ptr + 1,
                           (long)ims * hs, 0, 4, _stream));
  LSH_CALL(gemm_i8_i8o_dev_alpha(_qin.get(), _qweight.get(), _qout.get(), tok, ims, hs,
                                 _igemm_alpha.get(), _stream));
  // dropout.h:118-122: ReLU output goes through the unsigned (symmetry = false) quantiser
  const bool relu = _activation_fn == "relu";
  LSH_CALL(opb_quant_dropout_act_bias<T>(relu ? 1 : 0, nullptr, _ff2_inp.get(), nullptr, nullptr,
                                         nullptr, _qout.get(), _inter_b_ptr, _inter_cmax_ptr + 2,
                                         _output_cmax_ptr, (long)tok * ims, ims, 0.f, !relu,
                                         _stream));
  LSH_CALL(opb_fake_quantize<T>(nullptr, nullptr, _fake_weight.get(), _output_w_ptr,
                                _output_cmax_ptr + 1, (long)ims * hs, 4, true, _stream));
  LSH_CALL(gemm_f16_nt(_ff2_inp.get(), _fake_weight.get(), out_ptr, tok, hs, ims, _stream));
  LSH_CALL(opb_dropout_res_bias<T>(out_ptr, out_ptr, nullptr, _output_b_ptr, inp_ptr,
                                   (long)tok * hs, hs, 0.f, _stream));
  if (!_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(out_ptr, nullptr, nullptr, _vars.get(), nullptr, out_ptr,
                               _ffn_nw_ptr, _ffn_nb_ptr, nullptr, tok, hs, _stream));
}

// transformer_encoder_layer.cpp:277-293
template <typename T>
void TransformerEncoderLayer<T>::Forward(const T* input_ptr, const T* input_mask_ptr, T* out_ptr) {
  if (!input_ptr || !out_ptr) throw std::runtime_error("Forward: null input or output");
  if (!_attn_qkvw_ptr) throw std::runtime_error("Forward: no parameter blob assigned");
  if (_batch_tokens == 0) throw std::runtime_error("Forward: set_cur_batch_shape not called");
  if (_training)
    throw std::runtime_error("Forward: training mode (dropout, saved activations) is not provided");
  if (!_enable_quant)
    throw std::runtime_error("Forward: only the quantised path of the layer is provided");
  _stream = Context::Instance().get_stream();
  attn_layer_fw(input_ptr, input_mask_ptr, _ffn_inp.get());
  ffn_layer_fw(_ffn_inp.get(), out_ptr);
}

template class TransformerEncoderLayer<__half>;

}  // namespace hip
}  // namespace lightseq
