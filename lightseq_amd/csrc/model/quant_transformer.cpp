#include "quant_transformer.h"

namespace lightseq {
namespace hip {

QuantTransformer::QuantTransformer(const std::string weight_path, const int max_batch_size)
    : LSModel({"source_ids"}, {"target_ids", "target_scores"}), _max_batch_size(max_batch_size) {
  if (max_batch_size <= 0) throw std::runtime_error("max_batch_size must be positive");
  CHECK_GPU_ERROR(hipSetDevice(0));
  stream_.create();

  std::string res = tw_.initializing(weight_path);
  if (!res.empty()) throw std::runtime_error(res);
  if (tw_._sampling_method == "topk" || tw_._sampling_method == "topp") tw_._beam_size = 1;

  const size_t tokens = (size_t)_max_batch_size * tw_._max_step;
  d_input_.alloc(tokens);
  d_padding_mask_.alloc(tokens);
  d_encoder_output_.alloc(tokens * tw_._hidden_size);
  d_output_.alloc(tokens * std::max(tw_._beam_size, 1));

  encoder_ = std::make_shared<QuantBertEncoder>(max_batch_size, d_input_.get(),
                                                d_padding_mask_.get(), d_encoder_output_.get(),
                                                tw_.enc, stream_);
  res = encoder_->check();
  if (!res.empty()) throw std::runtime_error(res);
  decoder_ = std::make_shared<QuantDecoder>(max_batch_size, d_padding_mask_.get(),
                                            d_encoder_output_.get(), d_output_.get(), tw_,
                                            stream_, true);
  res = decoder_->check();
  if (!res.empty()) throw std::runtime_error(res);
  encoder_->init_buffer();
  decoder_->init_buffer();
  CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
  describe_input(0, kInt32, {_max_batch_size, tw_._max_step}, &encoder_->_p_d_token_id);
  describe_output(0, kInt32, {_max_batch_size, tw_._beam_size, tw_._max_step},
                  &decoder_->_p_d_result);
  describe_output(1, kFloat32, {_max_batch_size, tw_._beam_size},
                  &decoder_->_p_d_alive_seq_score);
}

QuantTransformer::~QuantTransformer() {
  decoder_.reset();
  encoder_.reset();  // before the buffers and the stream they use (members, released after this)
}

void QuantTransformer::Infer() {
  if (input_shapes_[0].size() != 2) throw std::runtime_error("source_ids must be 2-D");
  int batch_size = input_shapes_[0][0], seq_len = input_shapes_[0][1];
  if (tw_._multilg_type != 0) throw std::runtime_error("multilingle not supported");
  encoder_->run_one_infer(batch_size, seq_len);
  if (enc_out_tap_)
    CHECK_GPU_ERROR(hipMemcpyAsync(enc_out_tap_, d_encoder_output_.get(),
                                   (size_t)batch_size * seq_len * tw_._hidden_size * sizeof(__half),
                                   hipMemcpyDeviceToDevice, stream_));
  decoder_->run_one_infer(batch_size, seq_len);
  CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
  if (encoder_->finish_infer()) {  // an encoder route gave up and was switched off: once more
    encoder_->run_one_infer(batch_size, seq_len);
    decoder_->run_one_infer(batch_size, seq_len);
    CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
    encoder_->finish_infer();
  }
  encoder_->collect_profile();
  int output_seq_len = decoder_->_cur_step + 1;
  int output_k = decoder_->_output_topk ? tw_._beam_size : 1;
  set_output_shape(0, {batch_size, output_k, output_seq_len});
  set_output_shape(1, {batch_size, output_k});
}

void QuantTransformer::benchmark_mode(bool is_benchmark) {
  decoder_->benchmark_mode(is_benchmark);
}

LSMODEL_REGISTER(QuantTransformer)

}  // namespace hip
}  // namespace lightseq
