// extern "C" surface of the layer interface (include/lightseq_ops.h): the registry of layer
// objects by id that the reference keeps in pybind/pybind_layer.cpp:22-25, exceptions turned
// into status codes.
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../../../include/lightseq_ops.h"
#include "context.h"
#include "quant_linear_layer.h"
#include "transformer_decoder_layer.h"
#include "transformer_encoder_layer.h"

using namespace lightseq::hip;

namespace {

std::map<int, std::shared_ptr<TransformerEncoderLayer<__half>>> s_transformer_encoder_layers;
std::map<int, std::shared_ptr<TransformerDecoderLayer<__half>>> s_transformer_decoder_layers;
std::map<int, std::shared_ptr<QuantLinearLayer<__half>>> s_quant_linear_layers;

template <typename F>
int guarded(F&& f) {
  try {
    f();
    return LSH_OK;
  } catch (const std::exception& e) {
    return lsh::lsh_fail(LSH_ERR_INVALID, e.what());
  } catch (...) {
    return lsh::lsh_fail(LSH_ERR_INVALID, "unknown exception");
  }
}

template <typename M>
typename M::mapped_type find_layer(M& m, int id, const char* kind) {
  auto it = m.find(id);
  if (it == m.end())
    throw std::runtime_error(std::string(kind) + " #" + std::to_string(id) + " does not exist");
  return it->second;
}

}  // namespace

extern "C" {

int ls_layer_set_stream(lsh_stream_t stream) {
  Context::Instance().set_stream(reinterpret_cast<hipStream_t>(stream));
  return LSH_OK;
}

int ls_create_transformer_encoder_layer_fp16(int layer_id, int max_batch_tokens, int max_seq_len,
                                             int hidden_dim, int num_heads, int intermediate_size,
                                             float attn_prob_dropout_ratio,
                                             float activation_dropout_ratio,
                                             float hidden_dropout_ratio, int is_pre_ln,
                                             const char* activation_fn, int mask_future_tokens) {
  return guarded([&] {
    if (!activation_fn) throw std::runtime_error("activation_fn is null");
    s_transformer_encoder_layers[layer_id] = std::make_shared<TransformerEncoderLayer<__half>>(
        layer_id, max_batch_tokens, max_seq_len, hidden_dim, num_heads, intermediate_size,
        attn_prob_dropout_ratio, activation_dropout_ratio, hidden_dropout_ratio, is_pre_ln != 0,
        std::string(activation_fn), mask_future_tokens != 0);
  });
}

int ls_transformer_encoder_layer_fw_fp16(int layer_id, const void* input, const void* input_mask,
                                         void* output, int batch_size, int seq_len,
                                         int training_mode, int prelayernorm, int quant_mode) {
  (void)prelayernorm;  // fixed at construction, as in the reference (the argument is unused there)
  return guarded([&] {
    auto layer = find_layer(s_transformer_encoder_layers, layer_id, "Encoder layer");
    layer->set_cur_batch_shape(batch_size, seq_len);
    layer->SetTrainingMode(training_mode != 0);
    layer->SetQuantMode(quant_mode != 0);
    layer->Forward(reinterpret_cast<const __half*>(input),
                   reinterpret_cast<const __half*>(input_mask), reinterpret_cast<__half*>(output));
  });
}

int ls_create_transformer_decoder_layer_fp16(int layer_id, int max_batch_tokens, int max_seq_len,
                                             int hidden_dim, int num_heads, int intermediate_size,
                                             float attn_prob_dropout_ratio,
                                             float activation_dropout_ratio,
                                             float hidden_dropout_ratio, int is_pre_ln,
                                             const char* activation_fn) {
  return guarded([&] {
    if (!activation_fn) throw std::runtime_error("activation_fn is null");
    s_transformer_decoder_layers.erase(layer_id);  // a replaced layer leaves the shared count first
    s_transformer_decoder_layers[layer_id] = std::make_shared<TransformerDecoderLayer<__half>>(
        layer_id, max_batch_tokens, max_seq_len, hidden_dim, num_heads, intermediate_size,
        attn_prob_dropout_ratio, activation_dropout_ratio, hidden_dropout_ratio, is_pre_ln != 0,
        std::string(activation_fn));
  });
}

int ls_transformer_decoder_layer_fw_fp16(int layer_id, const void* dec_input,
                                         const void* enc_output, const void* enc_mask,
                                         void* dec_output, int batch_size, int trg_seq_len,
                                         int src_seq_len, int step, void* const* cache,
                                         int training_mode, int prelayernorm, int quant_mode) {
  (void)prelayernorm;  // fixed at construction, as in the reference (the argument is unused there)
  return guarded([&] {
    auto layer = find_layer(s_transformer_decoder_layers, layer_id, "Decoder layer");
    std::vector<__half*> cache_vec;
    if (step >= 0) {
      if (!cache) throw std::runtime_error("a decoding step needs the cache pointers");
      for (int i = 0; i < 5; ++i) cache_vec.push_back(reinterpret_cast<__half*>(cache[i]));
    }
    layer->set_cur_batch_shape(batch_size, trg_seq_len, src_seq_len, step);
    layer->SetTrainingMode(training_mode != 0);
    layer->SetQuantMode(quant_mode != 0);
    layer->Forward(reinterpret_cast<const __half*>(dec_input),
                   reinterpret_cast<const __half*>(enc_output),
                   reinterpret_cast<const __half*>(enc_mask),
                   reinterpret_cast<__half*>(dec_output), cache_vec);
  });
}

int ls_layer_param_count(const char* layer_name, int layer_id, long long* count) {
  return guarded([&] {
    const std::string name = layer_name ? layer_name : "";
    if (!count) throw std::runtime_error("layer_param_count: null result pointer");
    if (name == "TransformerEncoderLayer")
      *count = (long long)find_layer(s_transformer_encoder_layers, layer_id, "Encoder layer")
                   ->param_count();
    else if (name == "TransformerDecoderLayer")
      *count = (long long)find_layer(s_transformer_decoder_layers, layer_id, "Decoder layer")
                   ->param_count();
    else
      throw std::runtime_error("layer_param_count: unknown layer name");
  });
}

int ls_assign_layer_weight_grad_fp16(const void* weights, void* grads, const char* layer_name,
                                     int layer_id) {
  (void)grads;
  return guarded([&] {
    const std::string name = layer_name ? layer_name : "";
    if (name == "TransformerEncoderLayer")
      find_layer(s_transformer_encoder_layers, layer_id, "Encoder layer")
          ->assign_weight_ptr(reinterpret_cast<const __half*>(weights));
    else if (name == "TransformerDecoderLayer")
      find_layer(s_transformer_decoder_layers, layer_id, "Decoder layer")
          ->assign_weight_ptr(reinterpret_cast<const __half*>(weights));
    else
      throw std::runtime_error("assign_layer_weight_grad: unknown layer name");
  });
}

int ls_create_quant_linear_layer_fp16(int layer_id, int in_features, int out_features,
                                      int max_batch_tokens) {
  return guarded([&] {
    s_quant_linear_layers[layer_id] = std::make_shared<QuantLinearLayer<__half>>(
        layer_id, in_features, out_features, max_batch_tokens);
  });
}

int ls_quant_linear_layer_fw_fp16(int layer_id, const void* inputs, const void* weight,
                                  const void* clip_max, void* outputs, int batch_size, int seq_len,
                                  int quant_mode) {
  return guarded([&] {
    auto layer = find_layer(s_quant_linear_layers, layer_id, "QuantLinearLayer");
    layer->set_cur_batch_shape(batch_size, seq_len);
    layer->SetQuantMode(quant_mode != 0);
    layer->Forward(reinterpret_cast<const __half*>(inputs), reinterpret_cast<const __half*>(weight),
                   reinterpret_cast<const __half*>(clip_max), reinterpret_cast<__half*>(outputs));
  });
}

int ls_destroy_layer(const char* layer_name, int layer_id) {
  return guarded([&] {
    const std::string name = layer_name ? layer_name : "";
    if (name == "TransformerEncoderLayer")
      s_transformer_encoder_layers.erase(layer_id);
    else if (name == "TransformerDecoderLayer")
      s_transformer_decoder_layers.erase(layer_id);
    else if (name == "QuantLinearLayer")
      s_quant_linear_layers.erase(layer_id);
    else
      throw std::runtime_error("destroy_layer: unknown layer name");
  });
}

}  // extern "C"
