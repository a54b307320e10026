// "QuantGpt" model: the int8 GPT stack behind the LSModel interface.  Mirrors
// lightseq/inference/pywrapper/quant_gpt.{h,cc}: input 0 "token_ids" int32
// [batch, seq_len]; output 0 "result" is, by the file's sampling_method, either the
// sampled ids int32 [batch, sampled_len] ("topk") or the perplexity float [batch] ("ppl").
#pragma once

#include <memory>

#include "ls_model.h"
#include "quant_gpt_encoder.h"

namespace lightseq {
namespace hip {

class QuantGpt : public LSModel {
 public:
  QuantGpt(const std::string weight_path, const int max_batch_size);
  ~QuantGpt();

  void Infer() override;
  void benchmark_mode(bool is_benchmark) override { encoder_->benchmark_mode(is_benchmark); }
  void* get_stream() override { return stream_.get(); }

  QuantGptEncoder* encoder() { return encoder_.get(); }
  const QuantGptWeight& weight() const { return tw_; }

 private:
  bool is_ppl() const { return tw_._sampling_method == "ppl"; }
  // owners first: released after the encoder, also when the constructor throws half way
  StreamOwner stream_;
  DeviceBuffer<int> d_input_, d_sample_id;
  DeviceBuffer<float> d_ppl;
  std::shared_ptr<QuantGptEncoder> encoder_;
  int _max_batch_size;
  QuantGptWeight tw_;
};

}  // namespace hip
}  // namespace lightseq
