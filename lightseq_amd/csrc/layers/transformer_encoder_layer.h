// Quantised transformer encoder layer behind the reference's layer interface
// (lightseq/csrc/layers/includes/transformer_encoder_layer.h:20-105): same constructor
// arguments, set_cur_batch_shape / assign_weight_ptr / SetTrainingMode / SetQuantMode /
// Forward, the same flat parameter blob.  Forward only, storage type fp16.
#pragma once

#include <string>

#include "../model/model_util.h"

namespace lightseq {
namespace hip {

template <typename T>
class TransformerEncoderLayer {
 public:
  TransformerEncoderLayer(int layer_id, int max_batch_tokens, int max_seq_len, int hidden_size,
                          int num_heads, int intermediate_size, float attn_prob_dropout_ratio,
                          float activation_dropout_ratio, float hidden_output_dropout_ratio,
                          bool pre_or_postLayerNorm, std::string activation_fn,
                          bool mask_future_tokens = false);

  void Forward(const T* input_ptr, const T* input_mask_ptr, T* out_ptr);

  void set_cur_batch_shape(int batch_size, int seq_len);
  void SetTrainingMode(bool training);
  void SetQuantMode(bool enable_quant);
  bool IsTrainingMode() const { return _training; }
  // transformer_encoder_layer.h:66-105: qkvw, qkvb, ow, ob, nw, nb, inter_w, inter_b,
  // output_w, output_b, ffn_nw, ffn_nb, then the clip values 3 (qkv: input, weight, output)
  // + 3 (attention output projection) + 3 (ffn1) + 2 (ffn2: input, weight) + 1 (kv cache).
  void assign_weight_ptr(const T* weights_ptr);
  size_t param_count() const;

 private:
  void attn_layer_fw(const T* input_ptr, const T* input_mask_ptr, T* output_ptr);
  void ffn_layer_fw(T* inp_ptr, T* out_ptr);

  const int _layer_id;
  const int _max_batch_tokens, _max_seq_len, _hidden_size, _heads, _intermediate_size;
  const bool _is_pre_ln;
  const std::string _activation_fn;
  const bool _mask_future_tokens;
  int _batch_size = 0, _seq_len = 0, _batch_tokens = 0;
  bool _training = true;
  bool _enable_quant = false;
  hipStream_t _stream = nullptr;

  // local device memory, sized once at the maximum shapes
  DeviceBuffer<T> _ln_out, _qkv, _attn_o_inp, _ffn_inp, _ff2_inp, _fake_weight, _vars;
  DeviceBuffer<int8_t> _qin, _qout, _qweight;
  DeviceBuffer<float> _igemm_alpha;

  const T* _attn_qkvw_ptr = nullptr;
  const T* _attn_qkvb_ptr = nullptr;
  const T* _attn_ow_ptr = nullptr;
  const T* _attn_ob_ptr = nullptr;
  const T* _attn_nw_ptr = nullptr;
  const T* _attn_nb_ptr = nullptr;
  const T* _inter_w_ptr = nullptr;
  const T* _inter_b_ptr = nullptr;
  const T* _output_w_ptr = nullptr;
  const T* _output_b_ptr = nullptr;
  const T* _ffn_nw_ptr = nullptr;
  const T* _ffn_nb_ptr = nullptr;
  const T* _attn_qkv_cmax_ptr = nullptr;
  const T* _attn_out_cmax_ptr = nullptr;
  const T* _inter_cmax_ptr = nullptr;
  const T* _output_cmax_ptr = nullptr;
  const T* _attn_qkv_cache_cmax_ptr = nullptr;
};

}  // namespace hip
}  // namespace lightseq
