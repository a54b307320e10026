// Host-side container of a QuantBert model file (quant_bert.proto): configuration,
// float vectors, raw uint8 kernels and the per-layer clip_max table.
//
// Mirrors lightseq/inference/proto/quant_bert_weight.{h,cc} (`initializing`,
// config fields, weight order, the 11-entry clip table per layer) with one
// deliberate difference: the stored uint8 kernels are kept as bytes instead of
// being dequantised to float and re-quantised at init; code = uint8 - 127 is what
// that round trip recovers (the fp16 rounding error is at most 0.06 code).
#pragma once

#include <stdint.h>

#include <string>
#include <vector>

namespace lightseq {
namespace hip {

struct QuantBertLayerWeight {
  std::vector<float> multihead_norm_scale, multihead_norm_bias;
  std::vector<uint8_t> multihead_project_kernel_qkv;  // [H, 3H]
  std::vector<float> multihead_project_bias_qkv;
  std::vector<uint8_t> multihead_project_kernel_output;  // [H, H]
  std::vector<float> multihead_project_bias_output;
  std::vector<float> ffn_norm_scale, ffn_norm_bias;
  std::vector<uint8_t> ffn_first_kernel;  // [H, I]
  std::vector<float> ffn_first_bias;
  std::vector<uint8_t> ffn_second_kernel;  // [I, H]
  std::vector<float> ffn_second_bias;
};

class QuantBertWeight {
 public:
  // Parses the file; returns "" on success, else a description of the problem
  // (same contract as the reference's initializing()).
  std::string initializing(const std::string& weight_path);

  std::vector<uint8_t> token_embedding;  // [vocab, H]
  std::vector<float> position_embedding, norm_scale, norm_bias;
  std::vector<QuantBertLayerWeight> layers;

  float _src_emb_clip_max = 0.f;
  // 11 per layer: w_qkv, w_out, w_ffn1, w_ffn2, ln1_out, attn_ctx, ln2_out, ffn_act,
  // qkv_gemm_out, outproj_gemm_out, ffn1_gemm_out
  std::vector<float> _enc_clip_max;
  // Entries per layer in _enc_clip_max and whether the token embedding is scaled by
  // sqrt(hidden): 11 / false for QuantBert; the encoder of QuantTransformer carries a
  // twelfth (unused) clip and scales (inference/model/quant_encoder.cc.cu:140, :242).
  int _clip_stride = 11;
  bool _scale_embedding = false;

  int _hidden_size = 0, _inner_size = 0, _max_step = 0, _src_vocab_size = 0, _n_enc_layer = 0;
  int _dim_per_head = 0, _head_num = 0, _padding_id = 0, _multilg_type = 0;
  const int _weight_per_enc_layer = 12;
  bool _is_post_ln = false, _use_gelu = false;
  const float _quant_range = 127.f;

 private:
  std::string parse_proto(const uint8_t* data, size_t size);
};

}  // namespace hip
}  // namespace lightseq
