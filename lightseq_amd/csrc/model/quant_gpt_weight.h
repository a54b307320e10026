// Host-side container of a QuantGpt model file (quant_gpt.proto).
//
// Mirrors lightseq/inference/proto/quant_gpt_weight.{h,cc} (`initializing`,
// proto_get_model_config :36-63, proto_parse_emb_wei :68-112, proto_parse_enc_wei
// :117-245): same config rules and error strings, 12 clip values per layer (the eleven
// of the encoder plus the K/V-cache clip).  The stored uint8 kernels are kept as bytes;
// the layers reuse QuantBertLayerWeight.  The token embedding is stored [hidden, vocab].
#pragma once

#include <stdint.h>

#include <string>
#include <vector>

#include "quant_bert_weight.h"

namespace lightseq {
namespace hip {

class QuantGptWeight {
 public:
  std::string initializing(const std::string& weight_path);

  std::vector<uint8_t> token_embedding;  // [hidden, vocab]
  std::vector<float> position_embedding, norm_scale, norm_bias;
  std::vector<QuantBertLayerWeight> layers;
  float _src_emb_clip_max = 0.f, _output_ln_clip_max = 0.f, _logits_clip_max = 0.f;
  // 12 per layer: w_qkv, w_out, w_ffn1, w_ffn2, ln1_out, attn_ctx, ln2_out, ffn_act,
  // qkv_gemm_out, outproj_gemm_out, ffn1_gemm_out, kv_cache
  std::vector<float> _enc_clip_max;

  int _hidden_size = 0, _inner_size = 0, _max_step = 0, _src_vocab_size = 0, _n_enc_layer = 0;
  int _dim_per_head = 0, _head_num = 0, _padding_id = 0;
  const int _weight_per_enc_layer = 12;
  // defaults of the reference (quant_gpt_weight.h:93-96)
  std::string _sampling_method = "topk";
  int _topk = 4;
  float _topp = 0.75f;
  int _eos_id = 0;
  int _extra_decode_length = 0;  // <= 0 in the file means max_step
  const float _quant_range = 127.f;

 private:
  std::string parse_proto(const uint8_t* data, size_t size);
};

}  // namespace hip
}  // namespace lightseq
