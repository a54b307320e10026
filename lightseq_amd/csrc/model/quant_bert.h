// "QuantBert" model: the int8 BERT encoder behind the LSModel interface.
// Mirrors lightseq/inference/pywrapper/quant_bert.{h,cc}: input 0 "token_ids"
// int32 [batch, seq_len]; output 0 "encoder_output" fp16 [batch, seq_len, hidden].
#pragma once

#include <memory>

#include "ls_model.h"
#include "quant_bert_encoder.h"

namespace lightseq {
namespace hip {

class QuantBert : public LSModel {
 public:
  QuantBert(const std::string weight_path, const int max_batch_size);
  ~QuantBert();

  void Infer() override;
  void benchmark_mode(bool) override {}
  void* get_stream() override { return stream_.get(); }

  QuantBertEncoder* encoder() { return encoder_.get(); }
  const QuantBertWeight& weight() const { return tw_; }

 private:
  // owners first: released after the encoder, also when the constructor throws half way
  StreamOwner stream_;
  DeviceBuffer<int> d_input_, d_padding_mask_;
  DeviceBuffer<__half> d_encoder_output_;
  std::shared_ptr<QuantBertEncoder> encoder_;
  int _max_batch_size;
  QuantBertWeight tw_;
};

}  // namespace hip
}  // namespace lightseq
