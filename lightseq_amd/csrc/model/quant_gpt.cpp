#include "quant_gpt.h"

namespace lightseq {
namespace hip {

QuantGpt::QuantGpt(const std::string weight_path, const int max_batch_size)
    : LSModel({"token_ids"}, {"result"}), _max_batch_size(max_batch_size) {
  if (max_batch_size <= 0) throw std::runtime_error("max_batch_size must be positive");
  CHECK_GPU_ERROR(hipSetDevice(0));
  stream_.create();

  std::string res = tw_.initializing(weight_path);
  if (!res.empty()) throw std::runtime_error(res);

  const size_t tokens = (size_t)_max_batch_size * tw_._max_step;
  d_input_.alloc(tokens);
  d_sample_id.alloc(tokens);
  d_ppl.alloc(_max_batch_size);

  encoder_ = std::make_shared<QuantGptEncoder>(max_batch_size, d_input_.get(), d_ppl.get(),
                                               d_sample_id.get(), tw_, stream_);
  res = encoder_->check();
  if (!res.empty()) throw std::runtime_error(res);
  encoder_->init_buffer();
  CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
  describe_input(0, kInt32, {_max_batch_size, tw_._max_step}, &encoder_->_p_d_token_id);
  // a file configured for perplexity returns one float per sequence, otherwise the sampled ids
  if (is_ppl()) describe_output(0, kFloat32, {_max_batch_size}, &encoder_->_p_d_ppl);
  else describe_output(0, kInt32, {_max_batch_size, tw_._max_step}, &encoder_->_p_d_sample_id);
}

QuantGpt::~QuantGpt() {
  encoder_.reset();  // before the buffers and the stream it uses (members, released after this)
}

void QuantGpt::Infer() {
  if (input_shapes_[0].size() != 2) throw std::runtime_error("token_ids must be 2-D");
  int batch_size = input_shapes_[0][0], seq_len = input_shapes_[0][1];
  if (is_ppl()) {
    encoder_->run_one_infer(batch_size, seq_len);
    CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
    set_output_shape(0, {batch_size});
  } else if (tw_._sampling_method == "topk" || tw_._sampling_method == "topp") {
    int sampled_seq_len = encoder_->run_one_sample(batch_size, seq_len);
    CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
    set_output_shape(0, {batch_size, sampled_seq_len});
  } else {
    throw std::runtime_error("Unsupported sampling_method");
  }
}

LSMODEL_REGISTER(QuantGpt)

}  // namespace hip
}  // namespace lightseq
