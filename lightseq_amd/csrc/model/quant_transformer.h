// "QuantTransformer" model: int8 encoder + int8 decoder with beam search behind the
// LSModel interface.  Mirrors lightseq/inference/pywrapper/quant_transformer.{h,cc}:
// input 0 "source_ids" int32 [batch, seq_len]; output 0 "target_ids" int32
// [batch, beam_size, out_len]; output 1 "target_scores" float [batch, beam_size]
// (the decoder is built with output_topk = true, :51-53).
#pragma once

#include <memory>

#include "ls_model.h"
#include "quant_bert_encoder.h"
#include "quant_decoder.h"

namespace lightseq {
namespace hip {

class QuantTransformer : public LSModel {
 public:
  QuantTransformer(const std::string weight_path, const int max_batch_size);
  ~QuantTransformer();

  void Infer() override;
  void benchmark_mode(bool is_benchmark) override;
  void* get_stream() override { return stream_.get(); }

  QuantBertEncoder* encoder() { return encoder_.get(); }
  QuantDecoder* decoder() { return decoder_.get(); }
  const QuantTransformerWeight& weight() const { return tw_; }
  // optional copy of the encoder output ([batch, seq_len, hidden] fp16) taken between
  // the encoder and the decoder of every Infer()
  void set_encoder_output_tap(__half* dst) { enc_out_tap_ = dst; }

 private:
  // owners first: the stream and the buffers outlive the encoder and decoder that use them,
  // and are released when the constructor throws half way (unsupported files are common)
  StreamOwner stream_;
  DeviceBuffer<int> d_input_, d_padding_mask_, d_output_;
  DeviceBuffer<__half> d_encoder_output_;
  std::shared_ptr<QuantBertEncoder> encoder_;
  std::shared_ptr<QuantDecoder> decoder_;
  __half* enc_out_tap_ = nullptr;
  int _max_batch_size;
  QuantTransformerWeight tw_;
};

}  // namespace hip
}  // namespace lightseq
