#include "quant_transformer_weight.h"

#include <fstream>
#include <iostream>

#include "pb_reader.h"

namespace lightseq {
namespace hip {

using lsh::PbField;
using lsh::PbReader;

static bool ends_with(const std::string& s, const std::string& suf) {
  return s.size() >= suf.size() && s.compare(s.size() - suf.size(), suf.size(), suf) == 0;
}

static void take_bytes(const PbField& f, std::vector<uint8_t>& out) {
  if (f.wire != 2) throw std::runtime_error("protobuf: bytes field expected");
  out.assign(f.data, f.data + f.size);
}

std::string QuantTransformerWeight::initializing(const std::string& weight_path,
                                                 bool only_decoder) {
  if (ends_with(weight_path, ".hdf5"))
    return "HDF5 model files are not supported by this build (no HDF5 library); "
           "export the model as protobuf (.pb)";
  if (!ends_with(weight_path, ".pb"))
    return "Unsupported weight extention for [" + weight_path +
           "]; Supported extensions: .pb, .hdf5\n";
  std::ifstream in(weight_path, std::ios::binary | std::ios::ate);
  if (!in) return "Parse weights from [" + weight_path + "] failed.";
  std::streamsize size = in.tellg();
  in.seekg(0);
  std::vector<uint8_t> buf((size_t)size);
  if (size > 0 && !in.read(reinterpret_cast<char*>(buf.data()), size))
    return "Parse weights from [" + weight_path + "] failed.";
  try {
    return parse_proto(buf.data(), buf.size(), only_decoder);
  } catch (const std::exception& e) {
    return "Parse weights from [" + weight_path + "] failed: " + e.what();
  }
}

namespace {

// One QuantEmbeddingLayer message (src or trg use the same schema).
struct EmbeddingBlock {
  std::vector<uint8_t> token_embedding, kernel_kv;
  std::vector<float> position_embedding, norm_scale, norm_bias, bias_kv, shared_bias, lang_emb,
      kernel_kv_clip_max;
  float emb_clip_max = 0.f, output_ln_clip_max = 0.f, logits_clip_max = 0.f;
  bool present = false;

  void parse(const PbField& f) {
    present = true;
    PbReader r(f);
    PbField g;
    while (r.next(g)) {
      switch (g.number) {
        case 1: take_bytes(g, token_embedding); break;
        case 2: g.append_floats(position_embedding); break;
        case 3: g.append_floats(norm_scale); break;
        case 4: g.append_floats(norm_bias); break;
        case 5: take_bytes(g, kernel_kv); break;
        case 6: g.append_floats(bias_kv); break;
        case 7: g.append_floats(shared_bias); break;
        case 8: g.append_floats(lang_emb); break;
        case 9: emb_clip_max = g.as_float(); break;
        case 10: g.append_floats(kernel_kv_clip_max); break;
        case 11: output_ln_clip_max = g.as_float(); break;
        case 12: logits_clip_max = g.as_float(); break;
        default: break;
      }
    }
  }
};

}  // namespace

std::string QuantTransformerWeight::parse_proto(const uint8_t* data, size_t size,
                                                bool only_decoder) {
  enc.layers.clear();
  enc._enc_clip_max.clear();
  dec_layers.clear();
  _dec_clip_max.clear();
  EmbeddingBlock src, trg;
  std::vector<std::vector<float>> enc_clips, dec_clips;  // indexed by field number - first clip
  bool have_conf = false;
  PbReader top(data, size);
  PbField f;
  while (top.next(f)) {
    if (f.number == 1) {
      src.parse(f);
    } else if (f.number == 3) {
      trg.parse(f);
    } else if (f.number == 2) {  // encoder_stack (repeated QuantEncoderLayer)
      enc.layers.emplace_back();
      enc_clips.emplace_back(12, 0.f);
      QuantBertLayerWeight& l = enc.layers.back();
      PbReader r(f);
      PbField g;
      while (r.next(g)) {
        switch (g.number) {
          case 1: g.append_floats(l.multihead_norm_scale); break;
          case 2: g.append_floats(l.multihead_norm_bias); break;
          case 3: take_bytes(g, l.multihead_project_kernel_qkv); break;
          case 4: g.append_floats(l.multihead_project_bias_qkv); break;
          case 5: take_bytes(g, l.multihead_project_kernel_output); break;
          case 6: g.append_floats(l.multihead_project_bias_output); break;
          case 7: g.append_floats(l.ffn_norm_scale); break;
          case 8: g.append_floats(l.ffn_norm_bias); break;
          case 9: take_bytes(g, l.ffn_first_kernel); break;
          case 10: g.append_floats(l.ffn_first_bias); break;
          case 11: take_bytes(g, l.ffn_second_kernel); break;
          case 12: g.append_floats(l.ffn_second_bias); break;
          default:
            if (g.number >= 13 && g.number <= 24) enc_clips.back()[g.number - 13] = g.as_float();
            break;
        }
      }
    } else if (f.number == 4) {  // decoder_stack (repeated QuantDecoderLayer)
      dec_layers.emplace_back();
      dec_clips.emplace_back(19, 0.f);
      QuantDecoderLayerWeight& l = dec_layers.back();
      PbReader r(f);
      PbField g;
      while (r.next(g)) {
        switch (g.number) {
          case 1: g.append_floats(l.self_norm_scale); break;
          case 2: g.append_floats(l.self_norm_bias); break;
          case 3: take_bytes(g, l.self_project_kernel_qkv); break;
          case 4: g.append_floats(l.self_project_bias_qkv); break;
          case 5: take_bytes(g, l.self_project_kernel_output); break;
          case 6: g.append_floats(l.self_project_bias_output); break;
          case 7: g.append_floats(l.encdec_norm_scale); break;
          case 8: g.append_floats(l.encdec_norm_bias); break;
          case 9: take_bytes(g, l.encdec_project_kernel_q); break;
          case 10: g.append_floats(l.encdec_project_bias_q); break;
          case 11: take_bytes(g, l.encdec_project_kernel_output); break;
          case 12: g.append_floats(l.encdec_project_bias_output); break;
          case 13: g.append_floats(l.ffn_norm_scale); break;
          case 14: g.append_floats(l.ffn_norm_bias); break;
          case 15: take_bytes(g, l.ffn_first_kernel); break;
          case 16: g.append_floats(l.ffn_first_bias); break;
          case 17: take_bytes(g, l.ffn_second_kernel); break;
          case 18: g.append_floats(l.ffn_second_bias); break;
          default:
            if (g.number >= 19 && g.number <= 37) dec_clips.back()[g.number - 19] = g.as_float();
            break;
        }
      }
    } else if (f.number == 5) {  // model_conf
      have_conf = true;
      PbReader r(f);
      PbField g;
      while (r.next(g)) {
        switch (g.number) {
          case 1: _head_num = g.as_int32(); break;
          case 2: _beam_size = g.as_int32(); break;
          case 3: _extra_decode_length = g.as_int32(); break;
          case 4: _length_penalty = g.as_float(); break;
          case 5: _padding_id = g.as_int32(); break;
          case 6: _start_id = g.as_int32(); break;
          case 7: _diverse_lambda = g.as_float(); break;
          case 8: _sampling_method = g.as_string(); break;
          case 9: _topp = g.as_float(); break;
          case 10: _topk = g.as_int32(); break;
          case 11: _end_id = g.as_int32(); break;
          case 12: _is_post_ln = g.as_bool(); break;
          case 13: _no_scale_embedding = g.as_bool(); break;
          case 14: _use_gelu = g.as_bool(); break;
          case 15: _multilg_type = g.as_int32(); break;
          default: break;
        }
      }
    }
  }
  if (!trg.present || !have_conf || dec_layers.empty() || (!only_decoder && !src.present))
    return "Parse weights failed: incomplete QuantTransformer message.";

  // ---- model config (quant_transformer_weight.cc:35-86) ----
  _hidden_size = (int)trg.norm_scale.size();
  if (_hidden_size <= 0) return "Wrong norm_scale_size !";
  _max_step = (int)(trg.position_embedding.size() / _hidden_size);
  _inner_size = (int)(dec_layers[0].ffn_first_kernel.size() / _hidden_size);
  if (!only_decoder) _src_vocab_size = (int)(src.token_embedding.size() / _hidden_size);
  _trg_vocab_size = (int)(trg.token_embedding.size() / _hidden_size);
  if (!only_decoder) _n_enc_layer = (int)enc.layers.size();
  _n_dec_layer = (int)dec_layers.size();
  if (_head_num <= 0 || _hidden_size % _head_num != 0)
    throw std::runtime_error("Wrong head_num: hidden_size " + std::to_string(_hidden_size) +
                             " % head_num " + std::to_string(_head_num) + " != 0.");
  _dim_per_head = _hidden_size / _head_num;
  if (_end_id == 0) _end_id = _trg_vocab_size - 1;
  if (_sampling_method.empty()) _sampling_method = "beam_search";
  if (_hidden_size % 4 != 0)
    return "hidden_size should be a multiple of 4 to avoid misaligned address in CUDA";

  const size_t H = (size_t)_hidden_size, I = (size_t)_inner_size;
  // ---- embeddings (:95-208) ----
  if (!only_decoder) {
    if (src.token_embedding.size() != (size_t)_src_vocab_size * H)
      return "Wrong token_embedding_size !";
    if (src.position_embedding.size() != (size_t)_max_step * H)
      return "Wrong position_embedding_size !";
    if (src.norm_scale.size() != H) return "Wrong norm_scale_size !";
    if (src.norm_bias.size() != H) return "Wrong norm_bias_size !";
  }
  if (trg.token_embedding.size() != (size_t)_trg_vocab_size * H)
    return "Wrong token_embedding_size !";
  if (trg.position_embedding.size() != (size_t)_max_step * H)
    return "Wrong position_embedding_size !";
  if (trg.norm_bias.size() != H) return "Wrong norm_bias_size !";
  if (trg.kernel_kv.size() != H * H * 2 * (size_t)_n_dec_layer)
    return "Wrong encode_output_project_kernel_kv_size !";
  if (trg.kernel_kv_clip_max.size() != (size_t)_n_dec_layer)
    return "Wrong encode_output_project_kernel_kv_clip_max_size !";
  if (trg.bias_kv.size() != H * 2 * (size_t)_n_dec_layer)
    return "Wrong encode_output_project_bias_kv_size !";
  if (trg.shared_bias.size() != (size_t)_trg_vocab_size) return "Wrong shared_bias_size !";

  // ---- encoder (:213-340) ----
  if (!only_decoder) {
    for (size_t i = 0; i < enc.layers.size(); ++i) {
      const QuantBertLayerWeight& l = enc.layers[i];
      if (l.multihead_norm_scale.size() != H) return "Wrong multihead_norm_scale_size !";
      if (l.multihead_norm_bias.size() != H) return "Wrong multihead_norm_bias_size !";
      if (l.multihead_project_kernel_qkv.size() != H * H * 3)
        return "Wrong multihead_project_kernel_qkv_size !";
      if (l.multihead_project_bias_qkv.size() != H * 3)
        return "Wrong multihead_project_bias_qkv_size !";
      if (l.multihead_project_kernel_output.size() != H * H)
        return "Wrong multihead_project_kernel_output_size !";
      if (l.multihead_project_bias_output.size() != H)
        return "Wrong multihead_project_bias_output_size !";
      if (l.ffn_norm_scale.size() != H) return "Wrong ffn_norm_scale_size !";
      if (l.ffn_norm_bias.size() != H) return "Wrong ffn_norm_bias_size !";
      if (l.ffn_first_kernel.size() != H * I) return "Wrong ffn_first_kernel_size !";
      if (l.ffn_first_bias.size() != I) return "Wrong ffn_first_bias_size !";
      if (l.ffn_second_kernel.size() != H * I) return "Wrong ffn_second_kernel_size !";
      if (l.ffn_second_bias.size() != H) return "Wrong ffn_second_bias_size !";
      for (int c = 0; c < 12; ++c) {
        // the twelfth value (ffn_second_output) is stored but never read by the engine
        if (c < 11 && !(enc_clips[i][c] > 0.f))
          return "missing or non-positive clip_max in encoder layer";
        enc._enc_clip_max.push_back(enc_clips[i][c]);
      }
    }
    if (!(src.emb_clip_max > 0.f)) return "missing or non-positive emb_clip_max";
    enc.token_embedding = std::move(src.token_embedding);
    enc.position_embedding = std::move(src.position_embedding);
    enc.norm_scale = std::move(src.norm_scale);
    enc.norm_bias = std::move(src.norm_bias);
    enc._src_emb_clip_max = src.emb_clip_max;
    enc._hidden_size = _hidden_size;
    enc._inner_size = _inner_size;
    enc._max_step = _max_step;
    enc._src_vocab_size = _src_vocab_size;
    enc._n_enc_layer = _n_enc_layer;
    enc._dim_per_head = _dim_per_head;
    enc._head_num = _head_num;
    enc._padding_id = _padding_id;
    enc._multilg_type = _multilg_type;
    enc._is_post_ln = _is_post_ln;
    enc._use_gelu = _use_gelu;
    enc._clip_stride = 12;
    enc._scale_embedding = true;  // quant_encoder.cc.cu:242 passes `true` unconditionally
  }

  // ---- decoder (:345-520) ----
  for (size_t i = 0; i < dec_layers.size(); ++i) {
    const QuantDecoderLayerWeight& l = dec_layers[i];
    if (l.self_norm_scale.size() != H) return "Wrong self_norm_scale size !";
    if (l.self_norm_bias.size() != H) return "Wrong self_norm_bias_size !";
    if (l.self_project_kernel_qkv.size() != H * H * 3)
      return "Wrong self_project_kernel_qkv size !";
    if (l.self_project_bias_qkv.size() != H * 3) return "Wrong self_project_bias_qkv size !";
    if (l.self_project_kernel_output.size() != H * H)
      return "Wrong self_project_kernel_output size !";
    if (l.self_project_bias_output.size() != H) return "Wrong self_project_bias_output size !";
    if (l.encdec_norm_scale.size() != H) return "Wrong encdec_norm_scale size !";
    if (l.encdec_norm_bias.size() != H) return "Wrong encdec_norm_bias_size !";
    if (l.encdec_project_kernel_q.size() != H * H) return "Wrong encdec_project_kernel_q size !";
    if (l.encdec_project_bias_q.size() != H) return "Wrong encdec_project_bias_q size !";
    if (l.encdec_project_kernel_output.size() != H * H)
      return "Wrong encdec_project_kernel_output size !";
    if (l.encdec_project_bias_output.size() != H)
      return "Wrong encdec_project_bias_output size !";
    if (l.ffn_norm_scale.size() != H) return "Wrong ffn_norm_scale_size !";
    if (l.ffn_norm_bias.size() != H) return "Wrong ffn_norm_bias_size !";
    if (l.ffn_first_kernel.size() != H * I) return "Wrong ffn_first_kernel_size !";
    if (l.ffn_first_bias.size() != I) return "Wrong ffn_first_bias_size !";
    if (l.ffn_second_kernel.size() != H * I) return "Wrong ffn_second_kernel_size !";
    if (l.ffn_second_bias.size() != H) return "Wrong ffn_second_bias_size !";
    for (int c = 0; c < 19; ++c) {
      // index 17 (ffn_second_output) is stored but never read by the engine
      if (c != 17 && !(dec_clips[i][c] > 0.f))
        return "missing or non-positive clip_max in decoder layer";
      _dec_clip_max.push_back(dec_clips[i][c]);
    }
  }
  if (!(trg.emb_clip_max > 0.f) || !(trg.output_ln_clip_max > 0.f) ||
      !(trg.logits_clip_max > 0.f))
    return "missing or non-positive clip_max in trg_embedding";
  for (float c : trg.kernel_kv_clip_max)
    if (!(c > 0.f)) return "missing or non-positive encode_output_project_kernel_kv_clip_max";
  trg_token_embedding = std::move(trg.token_embedding);
  trg_position_embedding = std::move(trg.position_embedding);
  trg_norm_scale = std::move(trg.norm_scale);
  trg_norm_bias = std::move(trg.norm_bias);
  encode_output_project_kernel_kv = std::move(trg.kernel_kv);
  encode_output_project_bias_kv = std::move(trg.bias_kv);
  shared_bias = std::move(trg.shared_bias);
  _encode_output_project_kernel_kv_clip_max = std::move(trg.kernel_kv_clip_max);
  _trg_emb_clip_max = trg.emb_clip_max;
  _output_ln_clip_max = trg.output_ln_clip_max;
  _logits_clip_max = trg.logits_clip_max;
  return "";
}

void QuantTransformerWeight::print_model_config() const {
  std::cout << "***model config***" << std::endl;
  std::cout << "encoder layers: " << _n_enc_layer << std::endl;
  std::cout << "decoder layers: " << _n_dec_layer << std::endl;
  std::cout << "hidden size: " << _hidden_size << std::endl;
  std::cout << "inner size: " << _inner_size << std::endl;
  std::cout << "head number: " << _head_num << std::endl;
  std::cout << "dim per head: " << _dim_per_head << std::endl;
  std::cout << "src vocab size: " << _src_vocab_size << std::endl;
  std::cout << "trg vocab size: " << _trg_vocab_size << std::endl;
  std::cout << "is_post_ln: " << _is_post_ln << std::endl;
  std::cout << "no_scale_embedding: " << _no_scale_embedding << std::endl;
  std::cout << "use_gelu: " << _use_gelu << std::endl;
  std::cout << "start_id: " << _start_id << std::endl;
  std::cout << "end_id: " << _end_id << std::endl;
  std::cout << "padding_id: " << _padding_id << std::endl;
  std::cout << "multilg_type: " << _multilg_type << std::endl;
  std::cout << std::endl;
  std::cout << "***generator config***" << std::endl;
  std::cout << "beam size: " << _beam_size << std::endl;
  std::cout << "max step: " << _max_step << std::endl;
  std::cout << "extra decode length(max decode length - src input length): "
            << _extra_decode_length << std::endl;
  std::cout << "length penalty: " << _length_penalty << std::endl;
  std::cout << "diverse lambda: " << _diverse_lambda << std::endl;
  std::cout << "sampling method: " << _sampling_method << std::endl;
  std::cout << "topk: " << _topk << std::endl;
  std::cout << "topp: " << _topp << std::endl;
}

}  // namespace hip
}  // namespace lightseq
