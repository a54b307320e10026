// Host-side container of a QuantTransformer model file (quant_transformer.proto):
// configuration, float vectors, raw uint8 kernels and the clip_max tables.
//
// Mirrors lightseq/inference/proto/quant_transformer_weight.{h,cc} (`initializing`,
// proto_get_model_config :35-86, proto_parse_emb_wei :95-208, proto_parse_enc_wei
// :213-340, proto_parse_dec_wei :345-520): same config rules (sizes derived from the
// tensors, trg_end_id 0 means vocab-1, empty sampling_method means beam_search), same
// error strings, 12 clip values per encoder layer and 19 per decoder layer in the
// reference's order.  As for QuantBert the stored uint8 kernels are kept as bytes.
#pragma once

#include <stdint.h>

#include <string>
#include <vector>

#include "quant_bert_weight.h"

namespace lightseq {
namespace hip {

struct QuantDecoderLayerWeight {
  std::vector<float> self_norm_scale, self_norm_bias;
  std::vector<uint8_t> self_project_kernel_qkv;  // [H, 3H]
  std::vector<float> self_project_bias_qkv;
  std::vector<uint8_t> self_project_kernel_output;  // [H, H]
  std::vector<float> self_project_bias_output;
  std::vector<float> encdec_norm_scale, encdec_norm_bias;
  std::vector<uint8_t> encdec_project_kernel_q;  // [H, H]
  std::vector<float> encdec_project_bias_q;
  std::vector<uint8_t> encdec_project_kernel_output;  // [H, H]
  std::vector<float> encdec_project_bias_output;
  std::vector<float> ffn_norm_scale, ffn_norm_bias;
  std::vector<uint8_t> ffn_first_kernel;  // [H, I]
  std::vector<float> ffn_first_bias;
  std::vector<uint8_t> ffn_second_kernel;  // [I, H]
  std::vector<float> ffn_second_bias;
};

class QuantTransformerWeight {
 public:
  std::string initializing(const std::string& weight_path, bool only_decoder = false);

  // encoder half in the form the encoder stack consumes (clip stride 12, scaled embedding)
  QuantBertWeight enc;

  // target embedding block
  std::vector<uint8_t> trg_token_embedding;  // [H, trg_vocab]: also the logits kernel
  std::vector<float> trg_position_embedding, trg_norm_scale, trg_norm_bias;
  std::vector<uint8_t> encode_output_project_kernel_kv;  // [H, n_dec_layer * 2 * H]
  std::vector<float> encode_output_project_bias_kv;      // [n_dec_layer, 2, H]
  std::vector<float> shared_bias;                        // [trg_vocab]
  std::vector<float> _encode_output_project_kernel_kv_clip_max;  // [n_dec_layer]
  float _trg_emb_clip_max = 0.f, _output_ln_clip_max = 0.f, _logits_clip_max = 0.f;

  std::vector<QuantDecoderLayerWeight> dec_layers;
  // 19 per layer: w_self_qkv, w_self_out, w_encdec_q, w_encdec_out, w_ffn1, w_ffn2,
  // self_ln_out, self_attn_ctx, encdec_ln_out, encdec_attn_ctx, ffn_ln_out, ffn_act,
  // self_qkv_gemm_out, self_out_gemm_out, encdec_q_gemm_out, encdec_out_gemm_out,
  // ffn1_gemm_out, ffn2_gemm_out, kv_cache
  std::vector<float> _dec_clip_max;

  int _hidden_size = 0, _inner_size = 0, _max_step = 0, _src_vocab_size = 0, _trg_vocab_size = 0;
  int _n_enc_layer = 0, _n_dec_layer = 0, _dim_per_head = 0, _head_num = 0;
  const int _weight_per_enc_layer = 12, _weight_per_dec_layer = 18;
  int _beam_size = 0, _extra_decode_length = 0, _padding_id = 0, _start_id = 0, _end_id = 0;
  int _topk = 0, _multilg_type = 0;
  float _length_penalty = 0.f, _diverse_lambda = 0.f, _topp = 0.f;
  std::string _sampling_method;
  bool _is_post_ln = false, _no_scale_embedding = false, _use_gelu = false;
  const float _quant_range = 127.f;

  void print_model_config() const;

 private:
  std::string parse_proto(const uint8_t* data, size_t size, bool only_decoder);
};

}  // namespace hip
}  // namespace lightseq
