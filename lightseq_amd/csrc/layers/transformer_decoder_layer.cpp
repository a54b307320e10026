// Forward pass of the quantised decoder layer
// (lightseq/csrc/layers/transformer_decoder_layer.cpp:91-547), built from this library's
// operator kernels.  What differs from the reference's sequence is only where kernels are
// fused: each attention core (scores, masked softmax, context, head merge) is one kernel, and
// the int8 GEMMs read their scale from device memory in the epilogue.
#include "transformer_decoder_layer.h"

#include <algorithm>

#include "context.h"

namespace lightseq {
namespace hip {

using namespace lsh;

template <typename T>
int TransformerDecoderLayer<T>::_shared_nlayer = 0;
template <typename T>
DeviceBuffer<T> TransformerDecoderLayer<T>::_shared_encdec_kv;
template <typename T>
DeviceBuffer<T> TransformerDecoderLayer<T>::_shared_kv_tmp;
template <typename T>
DeviceBuffer<T> TransformerDecoderLayer<T>::_shared_kv_weight;
template <typename T>
T* TransformerDecoderLayer<T>::_shared_infer_encdec_kv_ptr = nullptr;

template <typename T>
TransformerDecoderLayer<T>::TransformerDecoderLayer(
    int layer_id, int max_batch_tokens, int max_seq_len, int hidden_size, int num_heads,
    int intermediate_size, float attn_prob_dropout_ratio, float activation_dropout_ratio,
    float hidden_output_dropout_ratio, bool pre_or_postLayerNorm, std::string activation_fn)
    : _layer_id(layer_id),
      _max_batch_tokens(max_batch_tokens),
      _max_seq_len(max_seq_len),
      _hidden_size(hidden_size),
      _heads(num_heads),
      _intermediate_size(intermediate_size),
      _is_pre_ln(pre_or_postLayerNorm),
      _activation_fn(activation_fn) {
  (void)attn_prob_dropout_ratio;  // ratios only matter in training mode, which Forward rejects
  (void)activation_dropout_ratio;
  (void)hidden_output_dropout_ratio;
  if (layer_id < 0) throw std::runtime_error("TransformerDecoderLayer: negative layer id");
  if (max_batch_tokens <= 0 || max_seq_len <= 0 || hidden_size <= 0 || num_heads <= 0 ||
      intermediate_size <= 0)
    throw std::runtime_error("TransformerDecoderLayer: sizes must be positive");
  if (hidden_size % num_heads != 0)
    throw std::runtime_error("TransformerDecoderLayer: hidden_size % num_heads != 0");
  const int hd = hidden_size / num_heads;
  if (hd != 32 && hd != 64 && hd != 128)
    throw std::runtime_error("TransformerDecoderLayer: head dim must be 32, 64 or 128");
  if (hidden_size % 16 != 0 || intermediate_size % 16 != 0)
    throw std::runtime_error(
        "TransformerDecoderLayer: hidden and intermediate size must be multiples of 16");
  if (activation_fn != "relu" && activation_fn != "gelu")
    throw std::runtime_error("not supported activation: " + activation_fn);

  const size_t tok = (size_t)max_batch_tokens, hs = (size_t)hidden_size,
               ims = (size_t)intermediate_size;
  if (_is_pre_ln) _ln_out.alloc(tok * hs);
  _qkv.alloc(3 * tok * hs);
  _attn_o_inp.alloc(tok * hs);
  _encdec_inp.alloc(tok * hs);
  _encdec_q.alloc(tok * hs);
  _ffn_inp.alloc(tok * hs);
  _ff2_inp.alloc(tok * ims);
  _fake_weight.alloc(hs * ims);
  _vars.alloc(tok);
  _qin.alloc(tok * std::max(hs, ims));
  _qout.alloc(tok * std::max(3 * hs, ims));
  _qweight.alloc(std::max(3 * hs * hs, hs * ims));
  _igemm_alpha.alloc(tok);
  ++_shared_nlayer;  // transformer_decoder_layer.cpp:64
}

template <typename T>
TransformerDecoderLayer<T>::~TransformerDecoderLayer() {
  // The reference never takes a layer down; here the count follows the live layers, so that
  // one process can build a second stack after destroying the first.
  if (--_shared_nlayer == 0) {
    _shared_encdec_kv = DeviceBuffer<T>();
    _shared_kv_tmp = DeviceBuffer<T>();
    _shared_kv_weight = DeviceBuffer<T>();
    _shared_infer_encdec_kv_ptr = nullptr;
  }
}

template <typename T>
size_t TransformerDecoderLayer<T>::param_count() const {
  const size_t hs = _hidden_size, ims = _intermediate_size;
  size_t n = hs * hs * 3 + hs * 3 + hs * hs + 3 * hs     // self attention
             + hs * hs + hs + hs * hs + 3 * hs           // cross attention
             + hs * ims + ims + hs * ims + 3 * hs        // ffn
             + 3 * 6 + 5 + 1;                            // clip values
  if (_layer_id == 0) n += (size_t)_shared_nlayer * (hs * hs * 2 + hs * 2);
  return n;
}

template <typename T>
void TransformerDecoderLayer<T>::assign_weight_ptr(const T* weights_ptr) {
  if (!weights_ptr) throw std::runtime_error("assign_weight_ptr: null parameter blob");
  const size_t hs = _hidden_size, ims = _intermediate_size;
  const T* wptr = weights_ptr;
  _attn_qkvw_ptr = wptr; wptr += hs * hs * 3;
  _attn_qkvb_ptr = wptr; wptr += hs * 3;
  _attn_ow_ptr = wptr;   wptr += hs * hs;
  _attn_ob_ptr = wptr;   wptr += hs;
  _attn_nw_ptr = wptr;   wptr += hs;
  _attn_nb_ptr = wptr;   wptr += hs;
  _encdec_attn_qw_ptr = wptr; wptr += hs * hs;
  _encdec_attn_qb_ptr = wptr; wptr += hs;
  _encdec_attn_ow_ptr = wptr; wptr += hs * hs;
  _encdec_attn_ob_ptr = wptr; wptr += hs;
  _encdec_attn_nw_ptr = wptr; wptr += hs;
  _encdec_attn_nb_ptr = wptr; wptr += hs;
  _inter_w_ptr = wptr;   wptr += hs * ims;
  _inter_b_ptr = wptr;   wptr += ims;
  _output_w_ptr = wptr;  wptr += hs * ims;
  _output_b_ptr = wptr;  wptr += hs;
  _ffn_nw_ptr = wptr;    wptr += hs;
  _ffn_nb_ptr = wptr;    wptr += hs;
  _attn_qkv_cmax_ptr = wptr;       wptr += 3;
  _attn_out_cmax_ptr = wptr;       wptr += 3;
  _encdec_qkv_cmax_ptr = wptr;     wptr += 3;
  _encdec_out_cmax_ptr = wptr;     wptr += 3;
  _inter_cmax_ptr = wptr;          wptr += 3;
  _output_cmax_ptr = wptr;         wptr += 3;
  _encdec_kv_cmax_ptr = wptr;      wptr += 5;
  _attn_qkv_cache_cmax_ptr = wptr; wptr += 1;
  if (_layer_id == 0) {
    _encdec_attn_kvw_ptr = wptr; wptr += (size_t)_shared_nlayer * hs * hs * 2;
    _encdec_attn_kvb_ptr = wptr; wptr += (size_t)_shared_nlayer * hs * 2;
  } else {
    _encdec_attn_kvw_ptr = nullptr;
    _encdec_attn_kvb_ptr = nullptr;
    _encdec_kv_cmax_ptr = nullptr;
  }
}

template <typename T>
void TransformerDecoderLayer<T>::set_cur_batch_shape(int batch_size, int trg_seq_len,
                                                     int src_seq_len, int step) {
  if (batch_size <= 0 || trg_seq_len <= 0 || src_seq_len <= 0)
    throw std::runtime_error("set_cur_batch_shape: batch_size and lengths must be positive");
  if ((long)batch_size * trg_seq_len > _max_batch_tokens)
    throw std::runtime_error("Batch token numbers " +
                             std::to_string((long)batch_size * trg_seq_len) +
                             " exceeds the limit " + std::to_string(_max_batch_tokens) + ".");
  if ((long)batch_size * src_seq_len > _max_batch_tokens)
    throw std::runtime_error("Source token numbers " +
                             std::to_string((long)batch_size * src_seq_len) +
                             " exceeds the limit " + std::to_string(_max_batch_tokens) + ".");
  if (src_seq_len > _max_seq_len || (step < 0 ? trg_seq_len : step + 1) > _max_seq_len)
    throw std::runtime_error("Sequence length exceeds the limit " +
                             std::to_string(_max_seq_len) + ".");
  _batch_size = batch_size;
  _trg_seq_len = trg_seq_len;  // the beam size in a decoding step
  _src_seq_len = src_seq_len;
  _batch_tokens = batch_size * trg_seq_len;
  _predict = step >= 0;
  _step = _predict ? step : -1;
}

template <typename T>
void TransformerDecoderLayer<T>::SetTrainingMode(bool training) { _training = training; }

template <typename T>
void TransformerDecoderLayer<T>::SetQuantMode(bool enable_quant) { _enable_quant = enable_quant; }

template <typename T>
void TransformerDecoderLayer<T>::quant_linear(const T* inp, const T* w, const T* cmax,
                                              int out_features, int in_features) {
  const int tok = _batch_tokens;
  LSH_CALL(opb_quantize<T>(_qin.get(), nullptr, _igemm_alpha.get(), inp, cmax,
                           (long)tok * in_features, tok, 2, _stream));
  LSH_CALL(opb_quantize<T>(_qweight.get(), nullptr, nullptr, w, cmax + 1,
                           (long)out_features * in_features, 0, 4, _stream));
  LSH_CALL(gemm_i8_i8o_dev_alpha(_qin.get(), _qweight.get(), _qout.get(), tok, out_features,
                                 in_features, _igemm_alpha.get(), _stream));
}

// transformer_decoder_layer.cpp:91-233
template <typename T>
void TransformerDecoderLayer<T>::self_attn_layer_fw(const T* input_ptr, T* output_ptr,
                                                    const std::vector<T*>& cache) {
  const int tok = _batch_tokens, hs = _hidden_size, hd = hs / _heads;
  const int from_len = _predict ? 1 : _trg_seq_len;
  const int to_len = _predict ? _step + 1 : _trg_seq_len;
  const int batch_size = _predict ? _batch_size * _trg_seq_len : _batch_size;
  if (_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(_ln_out.get(), nullptr, nullptr, _vars.get(), nullptr, input_ptr,
                               _attn_nw_ptr, _attn_nb_ptr, nullptr, tok, hs, _stream));
  quant_linear(_is_pre_ln ? _ln_out.get() : input_ptr, _attn_qkvw_ptr, _attn_qkv_cmax_ptr, 3 * hs,
               hs);
  // k and v leave this kernel as the cache will hold them: fake-quantised (:134-138)
  LSH_CALL(opb_quant_bias_add_transform_20314<T>(_qkv.get(), nullptr, _qout.get(), _attn_qkvb_ptr,
                                                 _attn_qkv_cmax_ptr + 2, batch_size, from_len, 3,
                                                 _heads, hd, _stream, _attn_qkv_cache_cmax_ptr));
  const size_t batch_dim = (size_t)tok * hs;
  const T* q_tf = _qkv.get();
  const T* k_tf = q_tf + batch_dim;
  const T* v_tf = k_tf + batch_dim;
  if (_predict) {  // :173-180: new cache = previous cache ++ this step's k / v
    LSH_CALL(opb_concat3_dim1<T>(cache[2], k_tf, cache[0], batch_size * _heads, hd, _step, 1,
                                 _stream));
    LSH_CALL(opb_concat3_dim1<T>(cache[3], v_tf, cache[1], batch_size * _heads, hd, _step, 1,
                                 _stream));
    k_tf = cache[0];
    v_tf = cache[1];
  }
  // scores, softmax (future positions masked outside a decoding step), context, head merge
  LSH_CALL(layer_cross_attention_f16(q_tf, k_tf, v_tf, nullptr, _attn_o_inp.get(), batch_size,
                                     from_len, to_len, _heads, hd, !_predict, _stream));

  quant_linear(_attn_o_inp.get(), _attn_ow_ptr, _attn_out_cmax_ptr, hs, hs);
  LSH_CALL(opb_quant_dropout_res_bias<T>(output_ptr, nullptr, _qout.get(), _attn_out_cmax_ptr + 2,
                                         _attn_ob_ptr, input_ptr, (long)tok * hs, hs, 0.f,
                                         _stream));
  if (!_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(output_ptr, nullptr, nullptr, _vars.get(), nullptr, output_ptr,
                               _attn_nw_ptr, _attn_nb_ptr, nullptr, tok, hs, _stream));
}

// transformer_decoder_layer.cpp:236-262: k and v of the encoder output for every decoder
// layer in one fp16 product with fake-quantised weights (the input is not quantised)
template <typename T>
void TransformerDecoderLayer<T>::encdec_kv_fw(const T* enc_output_ptr) {
  if (!enc_output_ptr) throw std::runtime_error("Forward: null encoder output");
  if (!_encdec_attn_kvw_ptr)
    throw std::runtime_error("Forward: layer 0 holds no cross-attention k/v weights");
  const size_t hs = _hidden_size;
  const int nl = _shared_nlayer, src_tok = _batch_size * _src_seq_len;
  const size_t kv_elems = (size_t)nl * 2 * _max_batch_tokens * hs;
  if (_shared_kv_tmp.size() != kv_elems) _shared_kv_tmp.alloc(kv_elems);
  if (!_predict && _shared_encdec_kv.size() != kv_elems) _shared_encdec_kv.alloc(kv_elems);
  if (_shared_kv_weight.size() != (size_t)nl * 2 * hs * hs)
    _shared_kv_weight.alloc((size_t)nl * 2 * hs * hs);
  LSH_CALL(opb_fake_quantize<T>(nullptr, nullptr, _shared_kv_weight.get(), _encdec_attn_kvw_ptr,
                                _encdec_kv_cmax_ptr + 1, (long)nl * 2 * hs * hs, 4, true,
                                _stream));
  LSH_CALL(gemm_f16_nt(enc_output_ptr, _shared_kv_weight.get(), _shared_kv_tmp.get(), src_tok,
                       nl * 2 * (int)hs, (int)hs, _stream));
  // [batch, src_len, layers * 2, heads, head_dim] -> [layers * 2, batch, heads, src_len, head_dim]
  LSH_CALL(opb_bias_add_transform_20314<T>(
      _predict ? _shared_infer_encdec_kv_ptr : _shared_encdec_kv.get(), _shared_kv_tmp.get(),
      _encdec_attn_kvb_ptr, _batch_size, _src_seq_len, nl * 2, _heads, (int)hs / _heads, _stream));
}

// transformer_decoder_layer.cpp:278-412
template <typename T>
void TransformerDecoderLayer<T>::encdec_attn_layer_fw(const T* input_ptr, const T* enc_mask_ptr,
                                                      T* output_ptr) {
  const int tok = _batch_tokens, hs = _hidden_size, hd = hs / _heads;
  if (_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(_ln_out.get(), nullptr, nullptr, _vars.get(), nullptr, input_ptr,
                               _encdec_attn_nw_ptr, _encdec_attn_nb_ptr, nullptr, tok, hs,
                               _stream));
  quant_linear(_is_pre_ln ? _ln_out.get() : input_ptr, _encdec_attn_qw_ptr, _encdec_qkv_cmax_ptr,
               hs, hs);
  LSH_CALL(opb_quant_bias_add_transform_20314<T>(
      _encdec_q.get(), nullptr, _qout.get(), _encdec_attn_qb_ptr, _encdec_qkv_cmax_ptr + 2,
      _batch_size, _trg_seq_len, 1, _heads, hd, _stream, nullptr));

  const T* kv = _predict ? _shared_infer_encdec_kv_ptr : _shared_encdec_kv.get();
  if (!kv) throw std::runtime_error("Forward: layer 0 has not produced the cross-attention k/v");
  const size_t src_dim = (size_t)_batch_size * _src_seq_len * hs;
  const T* k = kv + (size_t)_layer_id * 2 * src_dim;
  LSH_CALL(layer_cross_attention_f16(_encdec_q.get(), k, k + src_dim, enc_mask_ptr,
                                     _attn_o_inp.get(), _batch_size, _trg_seq_len, _src_seq_len,
                                     _heads, hd, false, _stream));

  quant_linear(_attn_o_inp.get(), _encdec_attn_ow_ptr, _encdec_out_cmax_ptr, hs, hs);
  LSH_CALL(opb_quant_dropout_res_bias<T>(output_ptr, nullptr, _qout.get(),
                                         _encdec_out_cmax_ptr + 2, _encdec_attn_ob_ptr, input_ptr,
                                         (long)tok * hs, hs, 0.f, _stream));
  if (!_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(output_ptr, nullptr, nullptr, _vars.get(), nullptr, output_ptr,
                               _encdec_attn_nw_ptr, _encdec_attn_nb_ptr, nullptr, tok, hs,
                               _stream));
}

// transformer_decoder_layer.cpp:415-483
template <typename T>
void TransformerDecoderLayer<T>::ffn_layer_fw(T* inp_ptr, T* out_ptr) {
  const int tok = _batch_tokens, hs = _hidden_size, ims = _intermediate_size;
  if (_is_pre_ln)
    LSH_CALL(opb_layer_norm<T>(_ln_out.get(), nullptr, nullptr, _vars.get(), nullptr, inp_ptr,
                               _ffn_nw_ptr, _ffn_nb_ptr, nullptr, tok, hs, _stream));
  quant_linear(_is_pre_ln ? _ln_out.get() : inp_ptr, _inter_w_ptr, _inter_cmax_ptr, ims, hs);
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

// transformer_decoder_layer.cpp:508-547
template <typename T>
void TransformerDecoderLayer<T>::Forward(const T* dec_input_ptr, const T* enc_output_ptr,
                                         const T* enc_mask_ptr, T* dec_output_ptr,
                                         const std::vector<T*>& cache) {
  if (!dec_input_ptr || !dec_output_ptr) throw std::runtime_error("Forward: null input or output");
  if (!_attn_qkvw_ptr) throw std::runtime_error("Forward: no parameter blob assigned");
  if (_batch_tokens == 0) throw std::runtime_error("Forward: set_cur_batch_shape not called");
  if (_training)
    throw std::runtime_error("Forward: training mode (dropout, saved activations) is not provided");
  if (!_enable_quant)
    throw std::runtime_error("Forward: only the quantised path of the layer is provided");
  if (_predict) {
    if (cache.size() < (_layer_id == 0 ? 5u : 4u))
      throw std::runtime_error("Forward: a decoding step needs the cache pointers");
    if (!cache[0] || !cache[1] || (_step > 0 && (!cache[2] || !cache[3])) ||
        (_layer_id == 0 && !cache[4]))
      throw std::runtime_error("Forward: null cache pointer");
  }
  _stream = Context::Instance().get_stream();

  if (_layer_id == 0) {
    if (_predict) {
      _shared_infer_encdec_kv_ptr = cache[4];
      if (_step == 0) encdec_kv_fw(enc_output_ptr);
    } else {
      encdec_kv_fw(enc_output_ptr);
    }
  }
  self_attn_layer_fw(dec_input_ptr, _encdec_inp.get(), cache);
  encdec_attn_layer_fw(_encdec_inp.get(), enc_mask_ptr, _ffn_inp.get());
  ffn_layer_fw(_ffn_inp.get(), dec_output_ptr);
}

template class TransformerDecoderLayer<__half>;

}  // namespace hip
}  // namespace lightseq
