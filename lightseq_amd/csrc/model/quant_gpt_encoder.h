// Host orchestration of the int8 GPT decoder-only stack on one MI355X: prompt pass,
// cached generation steps with greedy sampling, and perplexity.
//
// Same role and call order as lightseq/inference/model/quant_gpt_encoder.{h,cc.cu}
// (init_buffer :65-222, check :227-251, run_one_infer :253-291, run_one_sample
// :299-397, sample_one_token(_with_cache) :399-487, self_attention :470-560,
// self_attention_with_cache :563-643, ffn_add_norm(_with_cache) :646-776, compute_ppl
// :781-797), fp16 storage.  Differences in how the work is mapped to the GPU:
//  - keys / values live in caches of fixed stride [batch, head, max_step, d] and token
//    ids in [batch, max_step]; a step appends one column in place, where the reference
//    re-lays out every layer's cache and the whole id matrix per generated token;
//  - the prompt attention is one causal kernel (int8 scores on the MFMA units, softmax,
//    P.V, head merge and requantisation), a generation step's attention another;
//  - when sampling, vocabulary logits are computed for the last position only.
#pragma once

#include <string>
#include <vector>

#include "model_util.h"
#include "quant_gpt_weight.h"

namespace lightseq {
namespace hip {

class QuantGptEncoder {
 public:
  QuantGptEncoder(int max_batch_size, const int* p_d_token_id, float* p_d_ppl,
                  int* p_d_sample_id, const QuantGptWeight& tw, hipStream_t stream);
  ~QuantGptEncoder();
  void init_buffer();
  std::string check();
  void run_one_infer(int batch_size, int batch_seq_len);  // perplexity
  int run_one_sample(int batch_size, int batch_seq_len);  // returns the sampled length
  void benchmark_mode(bool is_benchmark) { _is_benchmark = is_benchmark; }
  // Random sampling (topk > 1, topp): restart the per-sequence generator states from `seed`
  // (0 at load; the reference seeds its cuRAND states with clock()).
  void set_seed(unsigned long long seed);

  // Optional record for parity checks: the last-position int8 logits of every sampling
  // step, [max_steps, batch, vocab] (device pointer owned by the caller).
  void set_step_record(int8_t* logits, int max_steps) {
    _rec_logits = logits;
    _rec_max_steps = max_steps;
  }
  int steps_run() const { return _steps_run; }
  // event times of the last run_one_sample: the prompt pass with the first token, the cached steps
  const PhaseEvents& phases() const { return _phases; }
  // Replay the cached steps through HIP graphs, one per (batch size, position): see StepGraphs.
  // Off while a step record is set.
  void graph_mode(bool on) { _use_graphs = on; }
  // copies of the intermediates of one layer at one cached step (names: see step_pass)
  StepTaps step_taps;
  int graphs_captured() const { return _graphs.captured(); }
  long graphs_replayed() const { return _graphs.replayed(); }
  int graph_nodes() const { return _graphs.last_graph_nodes(); }

  const int* _p_d_token_id;
  float* _p_d_ppl;
  int* _p_d_sample_id;

 private:
  void prompt_pass(const int* ids);
  const int8_t* step_pass();
  void ffn_add_norm(int rows, int8_t* in, int8_t* tmp);
  void enqueue_sampling(const int8_t* hidden, bool clear_flag);
  int finish_token();

  const int _max_batch_size;
  const QuantGptWeight& _tw;
  hipStream_t _stream;
  const float _quant_range = 127.f;
  const float _src_emb_clip_max, _output_ln_clip_max, _logits_clip_max;
  const std::vector<float> _enc_clip_max;
  const float _atten_scaler;
  bool _is_benchmark = false;
  bool _use_graphs = false;
  StepGraphs _graphs;

  int _batch_size = 0, _batch_seq_len = 0, _batch_token_num = 0, _batch_max_seq_len = 0;
  int _layer_id = 0, _steps_run = 0;
  PhaseEvents _phases;
  long _max_batch_dim;
  int* _h_unfinished = nullptr;  // pinned
  int8_t* _rec_logits = nullptr;
  int _tap_step = -2;  // the cached step being enqueued (tokens sampled so far), -2 outside one
  int _rec_max_steps = 0;

  DeviceBuffer<int> _real_seq_len, _ids, _last_ids, _unfinished;
  DeviceBuffer<long long> _sample_state;  // lsh_rng_state_t [max_batch_size]
  DeviceBuffer<__half> _query, _qkv_buf;  // q codes | k codes | v, each max_batch_dim
  DeviceBuffer<int8_t> _buf_a, _buf_b, _buf_q, _hid_last, _logits;
  DeviceBuffer<int32_t> _int32_ffn_out_buf;
  DeviceBuffer<int8_t> _self_k_cache, _self_v_cache;  // [n_layer][max_batch_dim]
  DeviceBuffer<int8_t> _int8_emb;                     // [vocab, H]
  DeviceBuffer<__half> _pos_emb, _out_ln_scale, _out_ln_bias;
  struct Layer {
    DeviceBuffer<int8_t> w_qkv, w_out, w_ffn1, w_ffn2;
    DeviceBuffer<int8_t> ffn1_act_lut;  // [inner, 256]: bias + GELU + requant per code
    DeviceBuffer<__half> ln1_scale, ln1_bias, b_qkv, b_out, ln2_scale, ln2_bias, b_ffn1, b_ffn2;
  };
  std::vector<Layer> _layers;
};

}  // namespace hip
}  // namespace lightseq
