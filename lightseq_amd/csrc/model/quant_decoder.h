// Host orchestration of the int8 transformer decoder with beam search on one MI355X.
//
// Same role, buffers and call order as lightseq/inference/model/quant_decoder.{h,cc.cu}
// (init_buffer :82-357, check :359-405, run_one_infer :413-484, project_encoder_output
// :489-515, run_step :520-566, embedding :571-590, decoder_stack :596-611,
// self_attention :617-723, encdec_attention :729-812, ffn_add_norm :815-935,
// beam_search :988-1075), fp16 storage.  What differs is how a step is mapped to the
// GPU: the int8 q.K scores, the softmax and the value sum run in one kernel, the
// encoder-decoder attention in another, the logits are searched by an exact per-row
// top-k plus a per-sentence merge (no global sort, no prefix scan), and the only
// device-to-host traffic of a step is the 4-byte finished-beam count that decides on
// early stop -- none at all in benchmark mode.
#pragma once

#include <string>
#include <vector>

#include "model_util.h"
#include "quant_transformer_weight.h"

namespace lightseq {
namespace hip {

class QuantDecoder {
 public:
  QuantDecoder(int max_batch_size, const int* p_d_padding_mask,
               const __half* p_d_encoder_output, int* p_d_result, QuantTransformerWeight& tw,
               hipStream_t stream, bool output_topk = false);
  ~QuantDecoder();
  void init_buffer();
  std::string check();
  void run_one_infer(int batch_size, int batch_seq_len);
  void benchmark_mode(bool is_benchmark) { _is_benchmark = is_benchmark; }
  // Restart the generator states of the sampling methods ("topk", "topp"): row i draws from
  // (seed, i).  Seed 0 at load.
  void set_seed(unsigned long long seed);

  // Optional per-step records for parity checks (device pointers owned by the caller):
  // logits [max_steps, batch*beam, vocab] int8 and the sequences after each step
  // [max_steps, batch*beam, max_step] int32.  steps_run() says how many were written.
  void set_step_record(int8_t* logits, int* alive_seq, int max_steps) {
    _rec_logits = logits;
    _rec_alive = alive_seq;
    _rec_max_steps = max_steps;
  }
  int steps_run() const { return _steps_run; }
  // event times of the last run_one_infer: the K/V projection of the encoder output, the steps
  const PhaseEvents& phases() const { return _phases; }
  // Replay decoding steps through HIP graphs, one per (batch, source length, step, buffer
  // parity): see StepGraphs.  Off while a step record is set.
  void graph_mode(bool on) { _use_graphs = on; }
  // copies of the intermediates of one layer at one step (names: see quant_decoder.cpp)
  StepTaps step_taps;
  int graphs_captured() const { return _graphs.captured(); }
  long graphs_replayed() const { return _graphs.replayed(); }
  int graph_nodes() const { return _graphs.last_graph_nodes(); }

  const int* _p_d_padding_mask;
  const __half* _p_d_encoder_output;
  int* _p_d_result;
  float* _p_d_alive_seq_score = nullptr;  // replaced by the caller's output buffer
  int _cur_step = 0;
  bool _output_topk;

 private:
  void project_encoder_output();
  bool run_step();
  void embedding();
  bool emb_ln_fused() const;
  void self_attention();
  void encdec_attention();
  void ffn_add_norm();
  void enqueue_step();
  void beam_search();
  void sample_tokens();
  bool step_runs_beam_search() const;

  const int _max_batch_size;
  QuantTransformerWeight& _tw;
  hipStream_t _stream;
  const float _quant_range = 127.f;
  const float _trg_emb_clip_max, _output_ln_clip_max, _logits_clip_max;
  const std::vector<float> _dec_clip_max;
  bool _is_benchmark = false;
  bool _use_graphs = false;
  StepGraphs _graphs;
  PhaseEvents _phases;

  int _batch_size = 0, _batch_seq_len = 0, _batch_token_num = 0, _step_token_num = 0;
  int _batch_max_decode_length = 0, _layer_id = 0, _steps_run = 0;
  long _layer_size_encdec_k, _layer_size_self_k;
  std::vector<float> _h_alive_seq_probs, _h_length_norm;
  int* _h_num_finished = nullptr;  // pinned; also receives the unfinished word of a sampling step
  bool _is_sampling = false;

  int8_t* _rec_logits = nullptr;
  int* _rec_alive = nullptr;
  int _rec_max_steps = 0;

  // activations and state
  DeviceBuffer<__half> _encdec_k, _encdec_v;      // [n_layer][max_batch*max_step*H]
  DeviceBuffer<__half> _encoder_out_buf;          // [tokens, n_layer*2*H]
  DeviceBuffer<__half> _cur_step_query, _query_buf1;
  DeviceBuffer<int8_t> _buf_a, _buf_b, _buf_q, _logits;
  DeviceBuffer<int32_t> _int32_ffn_out_buf;
  DeviceBuffer<int8_t> _self_k_cache[2], _self_v_cache[2];  // [n_layer][rows*max_step*H]
  int _cache_cur = 0;
  DeviceBuffer<int> _alive_seq[2];
  int _alive_cur = 0;
  DeviceBuffer<float> _alive_seq_probs, _alive_seq_score_own, _top_score, _topk_part_ws;
  DeviceBuffer<int> _top_idx, _parent, _num_finished;
  DeviceBuffer<int> _sample_unfinished;           // the flag of a sampling step
  DeviceBuffer<unsigned long long> _sample_state;  // lsh_rng_state_t per row (16 bytes each)
  // weights
  DeviceBuffer<int8_t> _int8_trg_emb;  // [vocab, H]: embedding rows and logits kernel
  DeviceBuffer<__half> _pos_emb, _out_ln_scale, _out_ln_bias, _kv_kernel /*[n_layer*2*H, H]*/,
      _kv_bias, _logit_bias;
  struct Layer {
    DeviceBuffer<int8_t> w_self_qkv, w_self_out, w_encdec_q, w_encdec_out, w_ffn1, w_ffn2;
    DeviceBuffer<int8_t> ffn1_act_lut;  // [inner, 256]: bias + activation + requant per code
    DeviceBuffer<__half> self_ln_scale, self_ln_bias, b_self_qkv, b_self_out, encdec_ln_scale,
        encdec_ln_bias, b_encdec_q, b_encdec_out, ffn_ln_scale, ffn_ln_bias, b_ffn1, b_ffn2,
        ffn2_colsum;
  };
  std::vector<Layer> _layers;
};

}  // namespace hip
}  // namespace lightseq
