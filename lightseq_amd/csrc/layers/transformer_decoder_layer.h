// Quantised transformer decoder layer behind the reference's layer interface
// (lightseq/csrc/layers/includes/transformer_decoder_layer.h:19-176): same constructor
// arguments as its Python binding passes (pybind/pybind_layer.cpp:110-132),
// set_cur_batch_shape / assign_weight_ptr / SetTrainingMode / SetQuantMode / Forward, the same
// flat parameter blob, the same cache convention of a decoding step.  Forward only, storage
// type fp16.
#pragma once

#include <string>
#include <vector>

#include "../model/model_util.h"

namespace lightseq {
namespace hip {

template <typename T>
class TransformerDecoderLayer {
 public:
  TransformerDecoderLayer(int layer_id, int max_batch_tokens, int max_seq_len, int hidden_size,
                          int num_heads, int intermediate_size, float attn_prob_dropout_ratio,
                          float activation_dropout_ratio, float hidden_output_dropout_ratio,
                          bool pre_or_postLayerNorm, std::string activation_fn);
  ~TransformerDecoderLayer();

  // cache (decoding step only, transformer_decoder_layer.cpp:173-189, :508-527 and
  // pybind_layer.cpp:160-176): [0] / [1] new self-attention k / v [batch * beam * heads,
  // step + 1, head_dim] (written), [2] / [3] the previous step's k / v [.., step, head_dim]
  // (read; null at step 0), [4] (layer 0 only) cross-attention k, v of all layers
  // [layers * 2, batch, heads, src_seq_len, head_dim] (written at step 0, read afterwards).
  void Forward(const T* dec_input_ptr, const T* enc_output_ptr, const T* enc_mask_ptr,
               T* dec_output_ptr, const std::vector<T*>& cache);

  // step < 0: the whole target sequence with future positions masked; step >= 0: one
  // decoding step, trg_seq_len is then the beam size (transformer_decoder_layer.h:67-92)
  void set_cur_batch_shape(int batch_size, int trg_seq_len, int src_seq_len, int step = -1);
  void SetTrainingMode(bool training);
  void SetQuantMode(bool enable_quant);
  // transformer_decoder_layer.h:103-170: qkvw, qkvb, ow, ob, nw, nb (self attention), qw, qb,
  // ow, ob, nw, nb (cross attention), inter_w, inter_b, output_w, output_b, ffn_nw, ffn_nb,
  // clip values 3 + 3 + 3 + 3 + 3 + 3 + 5 (cross k/v: input, weight, ...) + 1 (self k/v
  // cache); layer 0 is followed by the cross-attention k/v weights [layers * 2 * hidden,
  // hidden] and biases [layers * 2 * hidden] of every decoder layer created so far.
  void assign_weight_ptr(const T* weights_ptr);
  size_t param_count() const;
  static int shared_layer_count() { return _shared_nlayer; }

 private:
  void encdec_kv_fw(const T* enc_output_ptr);
  void self_attn_layer_fw(const T* input_ptr, T* output_ptr, const std::vector<T*>& cache);
  void encdec_attn_layer_fw(const T* input_ptr, const T* enc_mask_ptr, T* output_ptr);
  void ffn_layer_fw(T* inp_ptr, T* out_ptr);
  // int8 product of an activation and a weight matrix, both quantised here:
  // qout[tokens, out] = sat(alpha * quantize(inp) x quantize(w)^T), cmax = {input, weight, output}
  void quant_linear(const T* inp, const T* w, const T* cmax, int out_features, int in_features);

  const int _layer_id;
  const int _max_batch_tokens, _max_seq_len, _hidden_size, _heads, _intermediate_size;
  const bool _is_pre_ln;
  const std::string _activation_fn;
  int _batch_size = 0, _trg_seq_len = 0, _src_seq_len = 0, _batch_tokens = 0, _step = -1;
  bool _predict = false;
  bool _training = true;
  bool _enable_quant = false;
  hipStream_t _stream = nullptr;

  // decoder layers of the process share the cross-attention k/v (computed by layer 0)
  static int _shared_nlayer;
  static DeviceBuffer<T> _shared_encdec_kv, _shared_kv_tmp, _shared_kv_weight;
  static T* _shared_infer_encdec_kv_ptr;

  DeviceBuffer<T> _ln_out, _qkv, _attn_o_inp, _encdec_inp, _encdec_q, _ffn_inp, _ff2_inp,
      _fake_weight, _vars;
  DeviceBuffer<int8_t> _qin, _qout, _qweight;
  DeviceBuffer<float> _igemm_alpha;

  const T* _attn_qkvw_ptr = nullptr;
  const T* _attn_qkvb_ptr = nullptr;
  const T* _attn_ow_ptr = nullptr;
  const T* _attn_ob_ptr = nullptr;
  const T* _attn_nw_ptr = nullptr;
  const T* _attn_nb_ptr = nullptr;
  const T* _encdec_attn_qw_ptr = nullptr;
  const T* _encdec_attn_qb_ptr = nullptr;
  const T* _encdec_attn_ow_ptr = nullptr;
  const T* _encdec_attn_ob_ptr = nullptr;
  const T* _encdec_attn_nw_ptr = nullptr;
  const T* _encdec_attn_nb_ptr = nullptr;
  const T* _inter_w_ptr = nullptr;
  const T* _inter_b_ptr = nullptr;
  const T* _output_w_ptr = nullptr;
  const T* _output_b_ptr = nullptr;
  const T* _ffn_nw_ptr = nullptr;
  const T* _ffn_nb_ptr = nullptr;
  const T* _attn_qkv_cmax_ptr = nullptr;
  const T* _attn_out_cmax_ptr = nullptr;
  const T* _encdec_qkv_cmax_ptr = nullptr;
  const T* _encdec_out_cmax_ptr = nullptr;
  const T* _inter_cmax_ptr = nullptr;
  const T* _output_cmax_ptr = nullptr;
  const T* _encdec_kv_cmax_ptr = nullptr;
  const T* _attn_qkv_cache_cmax_ptr = nullptr;
  const T* _encdec_attn_kvw_ptr = nullptr;
  const T* _encdec_attn_kvb_ptr = nullptr;
};

}  // namespace hip
}  // namespace lightseq
