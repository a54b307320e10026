#include "quant_bert.h"

namespace lightseq {
namespace hip {

QuantBert::QuantBert(const std::string weight_path, const int max_batch_size)
    : LSModel({"token_ids"}, {"encoder_output"}), _max_batch_size(max_batch_size) {
  if (max_batch_size <= 0) throw std::runtime_error("max_batch_size must be positive");
  CHECK_GPU_ERROR(hipSetDevice(0));
  stream_.create();

  std::string res = tw_.initializing(weight_path);
  if (!res.empty()) throw std::runtime_error(res);

  const size_t tokens = (size_t)_max_batch_size * tw_._max_step;
  d_input_.alloc(tokens);
  d_padding_mask_.alloc(tokens);
  d_encoder_output_.alloc(tokens * tw_._hidden_size);

  encoder_ = std::make_shared<QuantBertEncoder>(max_batch_size, d_input_.get(),
                                                d_padding_mask_.get(), d_encoder_output_.get(),
                                                tw_, stream_);
  res = encoder_->check();
  if (!res.empty()) throw std::runtime_error(res);
  encoder_->init_buffer();
  CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
  describe_input(0, kInt32, {_max_batch_size, tw_._max_step}, &encoder_->_p_d_token_id);
  describe_output(0, kFloat16, {_max_batch_size, tw_._max_step, tw_._hidden_size},
                  &encoder_->_p_d_output);
}

QuantBert::~QuantBert() {
  encoder_.reset();  // before the buffers and the stream it uses (members, released after this)
}

void QuantBert::Infer() {
  if (input_shapes_[0].size() != 2) throw std::runtime_error("token_ids must be 2-D");
  int batch_size = input_shapes_[0][0], seq_len = input_shapes_[0][1];
  encoder_->run_one_infer(batch_size, seq_len);
  CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
  if (encoder_->finish_infer()) {  // a route gave up and was switched off: once more without it
    encoder_->run_one_infer(batch_size, seq_len);
    CHECK_GPU_ERROR(hipStreamSynchronize(stream_));
    encoder_->finish_infer();
  }
  encoder_->collect_profile();
  set_output_shape(0, {batch_size, seq_len, tw_._hidden_size});
}

LSMODEL_REGISTER(QuantBert)

}  // namespace hip
}  // namespace lightseq
