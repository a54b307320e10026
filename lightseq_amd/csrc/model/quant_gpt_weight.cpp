#include "quant_gpt_weight.h"

#include <fstream>

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

std::string QuantGptWeight::initializing(const std::string& weight_path) {
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
    return parse_proto(buf.data(), buf.size());
  } catch (const std::exception& e) {
    return "Parse weights from [" + weight_path + "] failed: " + e.what();
  }
}

std::string QuantGptWeight::parse_proto(const uint8_t* data, size_t size) {
  layers.clear();
  _enc_clip_max.clear();
  std::vector<std::vector<float>> clips;  // per layer, indexed by (field number - 13)
  bool have_emb = false, have_conf = false;
  int extra = 0;
  PbReader top(data, size);
  PbField f;
  while (top.next(f)) {
    if (f.number == 1) {  // src_embedding
      have_emb = true;
      PbReader r(f);
      PbField g;
      while (r.next(g)) {
        switch (g.number) {
          case 1: take_bytes(g, token_embedding); break;
          case 2: g.append_floats(position_embedding); break;
          case 3: g.append_floats(norm_scale); break;
          case 4: g.append_floats(norm_bias); break;
          case 5: _src_emb_clip_max = g.as_float(); break;
          case 6: _output_ln_clip_max = g.as_float(); break;
          case 7: _logits_clip_max = g.as_float(); break;
          default: break;
        }
      }
    } else if (f.number == 2) {  // encoder_stack (repeated)
      layers.emplace_back();
      clips.emplace_back(12, 0.f);
      QuantBertLayerWeight& l = layers.back();
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
            if (g.number >= 13 && g.number <= 24) clips.back()[g.number - 13] = g.as_float();
            break;
        }
      }
    } else if (f.number == 3) {  // model_conf
      have_conf = true;
      PbReader r(f);
      PbField g;
      while (r.next(g)) {
        switch (g.number) {
          case 1: _head_num = g.as_int32(); break;
          case 2: _padding_id = g.as_int32(); break;
          case 3: if (!g.as_string().empty()) _sampling_method = g.as_string(); break;
          case 4: if (g.as_float() != 0.f) _topp = g.as_float(); break;
          case 5: if (g.as_int32() != 0) _topk = g.as_int32(); break;
          case 6: if (g.as_int32() != 0) _eos_id = g.as_int32(); break;
          case 7: extra = g.as_int32(); break;
          default: break;
        }
      }
    }
  }
  if (!have_emb || !have_conf || layers.empty())
    return "Parse weights failed: incomplete QuantGpt message.";

  // model config (quant_gpt_weight.cc:36-63)
  _hidden_size = (int)norm_scale.size();
  if (_hidden_size <= 0) return "wrong norm_scale_size !";
  _inner_size = (int)(layers[0].ffn_first_kernel.size() / _hidden_size);
  _max_step = (int)(position_embedding.size() / _hidden_size);
  _src_vocab_size = (int)(token_embedding.size() / _hidden_size);
  _n_enc_layer = (int)layers.size();
  if (_head_num <= 0 || _hidden_size % _head_num != 0)
    throw std::runtime_error("Wrong head_num: hidden_size " + std::to_string(_hidden_size) +
                             " % head_num " + std::to_string(_head_num) + " != 0.");
  _dim_per_head = _hidden_size / _head_num;
  // the protobuf loader of the reference never reads extra_decode_length; its HDF5 loader
  // treats a non-positive value as max_step (quant_gpt_weight.cc:278-285)
  _extra_decode_length = extra > 0 ? extra : _max_step;

  const size_t H = (size_t)_hidden_size, I = (size_t)_inner_size;
  if (token_embedding.size() != (size_t)_src_vocab_size * H) return "wrong token_embedding_size !";
  if (position_embedding.size() != (size_t)_max_step * H) return "wrong position_embedding_size !";
  if (norm_bias.size() != H) return "wrong norm_bias_size !";
  for (size_t i = 0; i < layers.size(); ++i) {
    const QuantBertLayerWeight& l = layers[i];
    if (l.multihead_norm_scale.size() != H) return "wrong multihead_norm_scale_size !";
    if (l.multihead_norm_bias.size() != H) return "wrong multihead_norm_bias_size !";
    if (l.multihead_project_kernel_qkv.size() != H * H * 3)
      return "wrong multihead_project_kernel_qkv_size !";
    if (l.multihead_project_bias_qkv.size() != H * 3)
      return "wrong multihead_project_bias_qkv_size !";
    if (l.multihead_project_kernel_output.size() != H * H)
      return "wrong multihead_project_kernel_output_size !";
    if (l.multihead_project_bias_output.size() != H)
      return "wrong multihead_project_bias_output_size !";
    if (l.ffn_norm_scale.size() != H) return "wrong ffn_norm_scale_size !";
    if (l.ffn_norm_bias.size() != H) return "wrong ffn_norm_bias_size !";
    if (l.ffn_first_kernel.size() != H * I) return "wrong ffn_first_kernel_size !";
    if (l.ffn_first_bias.size() != I) return "wrong ffn_first_bias_size !";
    if (l.ffn_second_kernel.size() != H * I) return "wrong ffn_second_kernel_size !";
    if (l.ffn_second_bias.size() != H) return "wrong ffn_second_bias_size !";
    for (int c = 0; c < 12; ++c) {
      if (!(clips[i][c] > 0.f)) return "missing or non-positive clip_max in encoder layer";
      _enc_clip_max.push_back(clips[i][c]);
    }
  }
  if (!(_src_emb_clip_max > 0.f) || !(_output_ln_clip_max > 0.f) || !(_logits_clip_max > 0.f))
    return "missing or non-positive clip_max in src_embedding";
  return "";
}

}  // namespace hip
}  // namespace lightseq
