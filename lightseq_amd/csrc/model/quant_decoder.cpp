#include "quant_decoder.h"

#include "../ls_device.h"

#include <algorithm>

namespace lightseq {
namespace hip {

using namespace lsh;

static const float kMinLogProbability = -2000.f;  // inference/kernels/transformerKernels.h:12

QuantDecoder::QuantDecoder(int max_batch_size, const int* p_d_padding_mask,
                           const __half* p_d_encoder_output, int* p_d_result,
                           QuantTransformerWeight& tw, hipStream_t stream, bool output_topk)
    : _p_d_padding_mask(p_d_padding_mask),
      _p_d_encoder_output(p_d_encoder_output),
      _p_d_result(p_d_result),
      _output_topk(output_topk),
      _max_batch_size(max_batch_size),
      _tw(tw),
      _stream(stream),
      _trg_emb_clip_max(tw._trg_emb_clip_max),
      _output_ln_clip_max(tw._output_ln_clip_max),
      _logits_clip_max(tw._logits_clip_max),
      _dec_clip_max(tw._dec_clip_max),
      _layer_size_encdec_k((long)max_batch_size * tw._max_step * tw._hidden_size),
      _layer_size_self_k((long)max_batch_size * tw._max_step * tw._hidden_size * tw._beam_size),
      _h_alive_seq_probs((size_t)max_batch_size * std::max(tw._beam_size, 1),
                         kMinLogProbability / 2),
      _h_length_norm((size_t)std::max(tw._max_step, 1), 1.f) {
  // only the first beam of a sentence is alive before the first step (:64-66)
  for (size_t i = 0; i < _h_alive_seq_probs.size(); i += std::max(tw._beam_size, 1))
    _h_alive_seq_probs[i] = 0.f;
  if (tw._length_penalty >= 0)
    for (size_t i = 0; i < _h_length_norm.size(); i++)
      _h_length_norm[i] = length_norm((int)i + 1, tw._length_penalty);
}

QuantDecoder::~QuantDecoder() {
  if (_h_num_finished) (void)hipHostFree(_h_num_finished);
}

std::string QuantDecoder::check() {
  if (_tw._inner_size & 1) return "violate inner_size % 2 = 0";
  if (_tw._dim_per_head & 1) return "violate dim_per_head % 2 = 0";
  if (_tw._multilg_type != 0) return "multilingual models are not supported";
  if ((int)_tw.dec_layers.size() != _tw._n_dec_layer)
    return "violate p_d_dec_wei.size() = weight_per_dec_layer * n_dec_layer";
  if ((int)_dec_clip_max.size() != 19 * _tw._n_dec_layer) return "wrong clip_max table size";
  bool btmp = false;
  for (int i = 1; i < 64; i *= 2)
    if (i == _tw._beam_size) btmp = true;
  if (!btmp) return "wrong beam_size, should be 1, 2, 4, 8, 16 or 32";
  const std::string& m = _tw._sampling_method;
  if (m != "beam_search" && m != "topk" && m != "topp" && m != "topk_greedy")
    return std::string("unsupported sampling_method: ") + m;
  // (inference/model/quant_decoder.cc.cu:392-397)
  if (m == "topk" || m == "topp") _output_topk = false;
  if (m == "topk_greedy") _output_topk = true;
  if (m == "topk" && _tw._topk != 1 && _tw._topk != 2 && _tw._topk != 4 && _tw._topk != 8 &&
      _tw._topk != 16 && _tw._topk != 32)
    return "topk argument should be in [1,2,4,8,16,32]";
  if (m == "topp" && (!(_tw._topp > 0.f) || _tw._topp > 1.f)) return "topp outside (0, 1]";
  if (_tw._diverse_lambda != 0.f) return "diverse beam search is not available in this build";
  if (_tw._max_step > 1024) return "max_step should not greater than 1024";
  if (_tw._hidden_size % 16 != 0 || _tw._inner_size % 16 != 0)
    return "violate hidden_size % 16 = 0 and inner_size % 16 = 0 (int8 MFMA GEMM)";
  if (_tw._end_id < 0 || _tw._end_id >= _tw._trg_vocab_size || _tw._start_id < 0 ||
      _tw._start_id >= _tw._trg_vocab_size)
    return "start_id / end_id outside the target vocabulary";
  return "";
}

void QuantDecoder::init_buffer() {
  const int H = _tw._hidden_size, I = _tw._inner_size, L = _tw._n_dec_layer;
  const int V = _tw._trg_vocab_size, beam = _tw._beam_size;
  const size_t rows = (size_t)_max_batch_size * beam;
  const size_t tokens = (size_t)_max_batch_size * _tw._max_step;

  _encdec_k.alloc((size_t)L * _layer_size_encdec_k);
  _encdec_v.alloc((size_t)L * _layer_size_encdec_k);
  _encoder_out_buf.alloc(tokens * (size_t)L * 2 * H);
  _cur_step_query.alloc(rows * H);
  _query_buf1.alloc(rows * H);
  const size_t wide = rows * (size_t)std::max(I, 3 * H);
  _buf_a.alloc(wide);
  _buf_b.alloc(wide);
  _buf_q.alloc(wide);
  _logits.alloc(rows * (size_t)V);
  // up to 8 accumulator planes of the split-K second FFN product
  _int32_ffn_out_buf.alloc(rows * H * 8);
  for (int i = 0; i < 2; ++i) {
    _self_k_cache[i].alloc((size_t)L * _layer_size_self_k);
    _self_v_cache[i].alloc((size_t)L * _layer_size_self_k);
    CHECK_GPU_ERROR(hipMemsetAsync(_self_k_cache[i].get(), 0, _self_k_cache[i].size(), _stream));
    CHECK_GPU_ERROR(hipMemsetAsync(_self_v_cache[i].get(), 0, _self_v_cache[i].size(), _stream));
  }
  std::vector<int> start_id_vec(rows * _tw._max_step, _tw._start_id);
  for (int i = 0; i < 2; ++i) {
    _alive_seq[i].alloc(start_id_vec.size());
    _alive_seq[i].upload(start_id_vec.data(), start_id_vec.size(), _stream);
  }
  _alive_seq_probs.alloc(rows);
  _alive_seq_score_own.alloc(rows);
  CHECK_GPU_ERROR(hipMemsetAsync(_alive_seq_score_own.get(), 0, rows * sizeof(float), _stream));
  if (!_p_d_alive_seq_score) _p_d_alive_seq_score = _alive_seq_score_own.get();
  _top_score.alloc(rows * beam);
  _top_idx.alloc(rows * beam);
  // the per-row top-k dealt to several workgroups per row, where the vocabulary allows
  if (const size_t words = beam_search_step_workspace_words(_max_batch_size, beam, _tw._trg_vocab_size))
    _topk_part_ws.alloc(words);
  _parent.alloc(rows);
  _num_finished.alloc(1);
  _sample_unfinished.alloc(1);
  _sample_state.alloc(rows * 2);
  set_seed(0);
  CHECK_GPU_ERROR(hipHostMalloc(reinterpret_cast<void**>(&_h_num_finished), sizeof(int)));
  *_h_num_finished = 0;
  CHECK_GPU_ERROR(hipStreamSynchronize(_stream));  // start_id_vec dies below

  // ---- embedding block ----
  // stored [H, vocab]; one [vocab, H] copy serves the row lookup and the logits GEMM
  _int8_trg_emb = upload_kernel(_tw.trg_token_embedding, H, V, true, _stream);
  _pos_emb = upload_half(_tw.trg_position_embedding, _stream);
  _out_ln_scale = upload_half(_tw.trg_norm_scale, _stream);
  _out_ln_bias = upload_half(_tw.trg_norm_bias, _stream);
  _kv_bias = upload_half(_tw.encode_output_project_bias_kv, _stream);
  _logit_bias = upload_half(_tw.shared_bias, _stream);
  {
    // The K/V projection stays an fp16 GEMM (:497-501).  File layout [H, n_layer*2*H],
    // dequantised in flat chunks of 2*H*H with one clip each
    // (inference/proto/quant_transformer_weight.cc:144-160), then transposed to the
    // K-contiguous [n_layer*2*H, H] form of the GEMM here.
    const size_t kv_dim = (size_t)L * 2 * H, chunk = (size_t)2 * H * H;
    const std::vector<uint8_t>& src = _tw.encode_output_project_kernel_kv;
    std::vector<__half> t(kv_dim * H);
    for (size_t k = 0; k < (size_t)H; ++k)
      for (size_t n = 0; n < kv_dim; ++n) {
        const size_t flat = k * kv_dim + n;
        const float clip = _tw._encode_output_project_kernel_kv_clip_max[flat / chunk];
        // inference/tools/util.cc.cu:346-348
        const float v = ((float)src[flat] - _quant_range) * clip / _quant_range;
        t[n * H + k] = __float2half_rn(v);
      }
    _kv_kernel.alloc(t.size());
    _kv_kernel.upload(t.data(), t.size(), _stream);
    CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
  }

  // ---- layers ----
  _layers.clear();
  _layers.resize(L);
  for (int l = 0; l < L; ++l) {
    const QuantDecoderLayerWeight& w = _tw.dec_layers[l];
    Layer& d = _layers[l];
    d.self_ln_scale = upload_half(w.self_norm_scale, _stream);
    d.self_ln_bias = upload_half(w.self_norm_bias, _stream);
    d.b_self_qkv = upload_half(w.self_project_bias_qkv, _stream);
    d.b_self_out = upload_half(w.self_project_bias_output, _stream);
    d.encdec_ln_scale = upload_half(w.encdec_norm_scale, _stream);
    d.encdec_ln_bias = upload_half(w.encdec_norm_bias, _stream);
    d.b_encdec_q = upload_half(w.encdec_project_bias_q, _stream);
    d.b_encdec_out = upload_half(w.encdec_project_bias_output, _stream);
    d.ffn_ln_scale = upload_half(w.ffn_norm_scale, _stream);
    d.ffn_ln_bias = upload_half(w.ffn_norm_bias, _stream);
    d.b_ffn1 = upload_half(w.ffn_first_bias, _stream);
    d.b_ffn2 = upload_half(w.ffn_second_bias, _stream);
    d.w_self_qkv = upload_kernel(w.self_project_kernel_qkv, H, 3 * H, true, _stream);
    d.w_self_out = upload_kernel(w.self_project_kernel_output, H, H, true, _stream);
    d.w_encdec_q = upload_kernel(w.encdec_project_kernel_q, H, H, true, _stream);
    d.w_encdec_out = upload_kernel(w.encdec_project_kernel_output, H, H, true, _stream);
    d.w_ffn1 = upload_kernel(w.ffn_first_kernel, H, I, true, _stream);
    {
      const float* c = &_dec_clip_max[l * 19];
      d.ffn1_act_lut.alloc((size_t)I * 256);
      LSH_CALL(build_act_lut(d.ffn1_act_lut.get(), d.b_ffn1.get(), I, c[16] / _quant_range,
                             _quant_range / c[11], c[11],
                             _tw._use_gelu ? kActGelu : kActReluNarrow, _stream));
    }
    d.w_ffn2 = upload_kernel(w.ffn_second_kernel, I, H, true, _stream);
    if (!_tw._use_gelu) {
      // ReLU offset trick (:332-354): column sums of the fp16-rounded dequantised FFN2
      // kernel times clip/2
      const size_t n = w.ffn_second_kernel.size();
      DeviceBuffer<uint8_t> raw(n);
      raw.upload(w.ffn_second_kernel.data(), n, _stream);
      DeviceBuffer<__half> deq(n);
      LSH_CALL(stored_u8_dequant<__half>(raw.get(), deq.get(), (long)n, _dec_clip_max[l * 19 + 5],
                                         _stream));
      d.ffn2_colsum.alloc(H);
      LSH_CALL(scaled_colsum<__half>(deq.get(), d.ffn2_colsum.get(), I, H,
                                     _dec_clip_max[l * 19 + 11] / 2, _stream));
      CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
    }
  }
}

void QuantDecoder::set_seed(unsigned long long seed) {
  LSH_CALL(sample_state_setup(_sample_state.get(), (int)(_sample_state.size() / 2), seed, _stream));
}

// "topk_greedy" opens with one beam-search step, which gives every beam of a sentence another
// first token (inference/model/quant_decoder.cc.cu:1101-1106)
bool QuantDecoder::step_runs_beam_search() const {
  return !_is_sampling || (_tw._sampling_method == "topk_greedy" && _cur_step == 0);
}

void QuantDecoder::run_one_infer(int batch_size, int batch_seq_len) {
  if (batch_size > _max_batch_size)
    throw std::runtime_error("batch size of input greater than max_batch_size");
  if (batch_seq_len > _tw._max_step)
    throw std::runtime_error("seq len of input greater than max_step");
  if (batch_size <= 0 || batch_seq_len <= 0) throw std::runtime_error("empty input");

  /* ---step1. init--- */
  _batch_size = batch_size;
  _batch_seq_len = batch_seq_len;
  _batch_token_num = batch_size * batch_seq_len;
  _step_token_num = batch_size * _tw._beam_size;
  _batch_max_decode_length =
      std::min(_tw._max_step, batch_seq_len + _tw._extra_decode_length) - 1;
  // (:429-434)
  _is_sampling = _tw._sampling_method == "topk" || _tw._sampling_method == "topp" ||
                 _tw._sampling_method == "topk_greedy";
  if (_is_sampling) {
    _batch_max_decode_length = _tw._max_step;
    // nothing writes the scores of a sampled sequence; the reference hands its buffer to the
    // result writer as allocated, here every call starts it from zeros
    CHECK_GPU_ERROR(hipMemsetAsync(_alive_seq_score_own.get(), 0, sizeof(float) * _step_token_num,
                                   _stream));
  }
  _steps_run = 0;
  // every call starts from the same halves of the double-buffered sequences and caches (column
  // 0 of both sequence buffers holds the start token; everything else is rewritten as the
  // steps go), so that a step's launches are the same from call to call
  _alive_cur = 0;
  _cache_cur = 0;

  _phases.mark(0, _stream);
  project_encoder_output();
  CHECK_GPU_ERROR(hipMemcpyAsync(_alive_seq_probs.get(), _h_alive_seq_probs.data(),
                                 sizeof(float) * _step_token_num, hipMemcpyHostToDevice,
                                 _stream));

  /* ---step2. autoregressive decoding--- */
  _phases.mark(1, _stream);
  for (_cur_step = 0; _cur_step < _batch_max_decode_length - 1; _cur_step++) {
    bool early_stop = run_step();
    if (!_is_benchmark && early_stop) break;
  }
  _phases.mark(2, _stream);
  _phases.set_loop_steps(_steps_run);

  /* ---step3. output the decoding result--- */
  // The steps keep the scores of finished beams in the decoder's own buffer: a step may be a
  // recorded graph, and the caller may hand over another output buffer between two calls.
  if (_p_d_alive_seq_score != _alive_seq_score_own.get())
    CHECK_GPU_ERROR(hipMemcpyAsync(_p_d_alive_seq_score, _alive_seq_score_own.get(),
                                   sizeof(float) * _step_token_num, hipMemcpyDeviceToDevice,
                                   _stream));
  int* alive = _alive_seq[_alive_cur].get();
  if (_output_topk || _is_sampling) {
    if (_cur_step == _batch_max_decode_length) _cur_step -= 1;
    LSH_CALL(write_topk_result(alive, _p_d_alive_seq_score, _p_d_result, _tw._trg_vocab_size,
                               _tw._max_step, _tw._beam_size, _tw._end_id, _step_token_num,
                               _cur_step + 1, _stream));
    return;
  }
  if (_tw._length_penalty >= 0.f || _cur_step == _batch_max_decode_length) {
    LSH_CALL(write_trg_tokenid_pos_penalty(alive, _p_d_alive_seq_score, _p_d_result,
                                           _tw._max_step, _tw._beam_size, _batch_size,
                                           _cur_step + 1, _stream));
  } else {
    LSH_CALL(write_trg_tokenid_neg_penalty(alive, _p_d_alive_seq_score, _p_d_result,
                                           _tw._max_step, _tw._beam_size, _tw._trg_vocab_size,
                                           _tw._end_id, _batch_size, _cur_step + 1, _stream));
  }
}

void QuantDecoder::project_encoder_output() {
  const int H = _tw._hidden_size, L = _tw._n_dec_layer;
  const int kv_dim = H * 2 * L;
  LSH_CALL(gemm_f16_nt(_p_d_encoder_output, _kv_kernel.get(), _encoder_out_buf.get(),
                       _batch_token_num, kv_dim, H, _stream));
  // _encoder_out_buf: [batch_size, batch_seq_len, layer_num, 2, hidden_size]
  LSH_CALL(arrange_encdec_kv<__half>(_batch_token_num, L, H, _stream, _encoder_out_buf.get(),
                                     _kv_bias.get(), _encdec_k.get(), _encdec_v.get(),
                                     _layer_size_encdec_k, _batch_seq_len, _tw._dim_per_head,
                                     _tw._head_num));
}

bool QuantDecoder::run_step() {
  const bool search = step_runs_beam_search();
  // The launches of a step depend on the shapes of the call, the step index and which of the
  // two sequence / cache buffers is current: one graph per such key.  A sampling step clears
  // its flag with a memset and runs eagerly.
  const uint64_t key = ((uint64_t)_batch_size << 40) | ((uint64_t)_batch_seq_len << 24) |
                       ((uint64_t)_cur_step << 8) | (uint64_t)(_alive_cur << 1 | _cache_cur);
  _graphs.run(key, _stream,
              _use_graphs && !_is_sampling && !_rec_logits && !_rec_alive && !step_taps.any(),
              [&] { enqueue_step(); });
  ++_steps_run;
  if (!search) {
    // (:979-984, 1126-1131) the sequences stay in their buffer, the caches are not reordered
    if (_is_benchmark) return false;
    CHECK_GPU_ERROR(hipMemcpyAsync(_h_num_finished, _sample_unfinished.get(), sizeof(int),
                                   hipMemcpyDeviceToHost, _stream));
    CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
    return *_h_num_finished != 1;
  }
  _alive_cur ^= 1;
  if (_cur_step > 0) _cache_cur ^= 1;
  if (!_is_benchmark) {
    // the one device-to-host word of a step: all beams finished -> stop early
    CHECK_GPU_ERROR(hipMemcpyAsync(_h_num_finished, _num_finished.get(), sizeof(int),
                                   hipMemcpyDeviceToHost, _stream));
    CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
    if (*_h_num_finished == _step_token_num) return true;
  }
  return false;
}

// everything a step puts on the stream: embedding, the layer stack, the logits, the search
// and the cache reorder (kernels and device-to-device copies only, so that it can be captured)
void QuantDecoder::enqueue_step() {
  LnFewRowsScope few_rows;  // every step of every batch size: layer norms by the row kernel
  embedding();
  for (_layer_id = 0; _layer_id < _tw._n_dec_layer; _layer_id++) {
    self_attention();
    encdec_attention();
    ffn_add_norm();
  }
  /* --- Project hidden states to vocab logits (:527-532) --- */
  LSH_CALL(gemm_i8_i8o(_buf_a.get(), _int8_trg_emb.get(), _logits.get(), _step_token_num,
                       _tw._trg_vocab_size, _tw._hidden_size,
                       _output_ln_clip_max * _trg_emb_clip_max / (_logits_clip_max * _quant_range),
                       _stream));
  if (_rec_logits && _cur_step < _rec_max_steps)
    CHECK_GPU_ERROR(hipMemcpyAsync(
        _rec_logits + (size_t)_cur_step * _step_token_num * _tw._trg_vocab_size, _logits.get(),
        (size_t)_step_token_num * _tw._trg_vocab_size, hipMemcpyDeviceToDevice, _stream));
  if (step_runs_beam_search())
    beam_search();
  else
    sample_tokens();
}

// Step taps (debug): name -> what is copied, of layer step_taps' layer at its step.
//   self_ln_q, self_q, self_ctx_q, self_out_q, encdec_ln_q, encdec_ctx_q, encdec_out_q, ffn_ln_q,
//   next_ln_q: int8 [rows, hidden];  ffn1_act_q: int8 [rows, inner];  ffn2_acc: int32 [rows, hidden]
//   self_k_cache, self_v_cache: the layer's int8 caches [rows, heads, max_step, d] after the append
//   encdec_q: fp16 [batch, heads, beam, d];  encdec_k, encdec_v: fp16 [batch, heads, src_len, d]
//   res_in, res_self, res_encdec, res_out: the fp16 residual stream [rows, hidden] at the start of
//   the layer, after the first, the second and the last layer norm
#define TAP(name, ptr, bytes) step_taps.copy(_layer_id, _cur_step, name, ptr, bytes, _stream)

// hidden sizes the fused embedding + first layer norm covers
bool QuantDecoder::emb_ln_fused() const {
  return _tw._hidden_size % 4 == 0 && _tw._hidden_size <= 1024;
}

void QuantDecoder::embedding() {
  if (emb_ln_fused()) return;  // done by the first layer's launch
  LSH_CALL(dec_emb_i8I<__half>(_int8_trg_emb.get(), _pos_emb.get(), _alive_seq[_alive_cur].get(),
                               _cur_step_query.get(), _batch_size, _tw._beam_size,
                               _tw._hidden_size, _tw._trg_vocab_size, _cur_step, _tw._max_step,
                               _stream, _trg_emb_clip_max / _quant_range, true, true));
}

void QuantDecoder::self_attention() {
  const int H = _tw._hidden_size, M = _step_token_num;
  const Layer& w = _layers[_layer_id];
  const float* c = &_dec_clip_max[_layer_id * 19];
  const float Q = _quant_range;
  int8_t* k_cache = _self_k_cache[_cache_cur].get() + (size_t)_layer_id * _layer_size_self_k;
  int8_t* v_cache = _self_v_cache[_cache_cur].get() + (size_t)_layer_id * _layer_size_self_k;

  if (_layer_id == 0) {
    if (emb_ln_fused()) {
      // the step's embedding and the first layer norm in one launch (the bytes of the pair)
      LSH_CALL(dec_emb_norm_layer_i8O<__half>(
          _int8_trg_emb.get(), _pos_emb.get(), _alive_seq[_alive_cur].get(),
          _cur_step_query.get(), _buf_a.get(), w.self_ln_scale.get(), w.self_ln_bias.get(),
          w.b_self_out.get(), M, H, _tw._trg_vocab_size, _cur_step, _tw._max_step,
          _trg_emb_clip_max / _quant_range, true, Q / c[6], _tw._is_post_ln, _stream));
    } else {
      LSH_CALL(norm_layer_resual_i8O<__half>(M, H, _stream, _cur_step_query.get(), _buf_a.get(),
                                             w.self_ln_scale.get(), w.self_ln_bias.get(),
                                             w.b_self_out.get(), Q / c[6], _tw._is_post_ln));
    }
  }
  const size_t mh = (size_t)M * H;
  TAP("self_ln_q", _buf_a.get(), mh);
  TAP("res_in", _cur_step_query.get(), mh * sizeof(__half));
  const float attn_scale =
      __half2float(__float2half_rn(sqrtf(1.f / (float)_tw._dim_per_head)));
  // With taps set the two launches run, so that q and the caches are copied before the
  // attention as the tap names promise; the bytes are the same either way.
  if (!step_taps.any() && decself_qkv_attention_enabled() && _tw._dim_per_head == 64 &&
      decself_qkv_attention_supported(M, H, _tw._head_num, _tw._max_step)) {
    LSH_CALL(decself_qkv_attention_i8(_buf_a.get(), w.w_self_qkv.get(), w.b_self_qkv.get(),
                                      _buf_q.get(), k_cache, v_cache, _buf_b.get(), M, H,
                                      _tw._head_num, _tw._max_step, _cur_step,
                                      c[0] * c[6] / (c[12] * Q), c[12] / Q, Q / c[18], attn_scale,
                                      c[18] / Q, Q / c[7], _stream));
  } else {
  // QKV product; its epilogue is ker_arrange_decself_qkv_i8I_i8O: q -> _buf_q, k / v -> slot
  // _cur_step of the caches (all three with the cache clip)
  if (_tw._dim_per_head % 16 == 0) {
    LSH_CALL(gemm_i8_decself_qkv_i8o(_buf_a.get(), w.w_self_qkv.get(), w.b_self_qkv.get(),
                                     _buf_q.get(), k_cache, v_cache, M, H, H, _tw._head_num,
                                     _tw._max_step, _cur_step, c[0] * c[6] / (c[12] * Q),
                                     c[12] / Q, Q / c[18], _stream));
  } else {
    LSH_CALL(gemm_i8_i8o(_buf_a.get(), w.w_self_qkv.get(), _buf_b.get(), M, 3 * H, H,
                         c[0] * c[6] / (c[12] * Q), _stream));
    LSH_CALL(arrange_decself_qkv_i8I_i8O<__half>(M, H, _stream, _buf_b.get(), w.b_self_qkv.get(),
                                                 _buf_q.get(), k_cache, v_cache, _tw._head_num,
                                                 _tw._dim_per_head, _tw._max_step, _cur_step,
                                                 c[12] / Q, Q / c[18]));
  }
  TAP("self_q", _buf_q.get(), mh);
  TAP("self_k_cache", k_cache, mh * _tw._max_step);
  TAP("self_v_cache", v_cache, mh * _tw._max_step);
  // int8 q.K -> softmax -> new value, one kernel
  LSH_CALL(decself_attention_i8(_buf_q.get(), k_cache, v_cache, _buf_b.get(), M * _tw._head_num,
                                _cur_step + 1, _tw._max_step, _tw._head_num, _tw._dim_per_head,
                                attn_scale, c[18] / Q, Q / c[7], _stream));
  }
  TAP("self_ctx_q", _buf_b.get(), mh);
  LSH_CALL(gemm_i8_i8o(_buf_b.get(), w.w_self_out.get(), _buf_a.get(), M, H, H,
                       c[1] * c[7] / (c[13] * Q), _stream));
  TAP("self_out_q", _buf_a.get(), mh);
  LSH_CALL((residual_bias_ln_i8O<__half, int8_t>(
      _buf_a.get(), w.encdec_ln_scale.get(), w.encdec_ln_bias.get(), w.b_encdec_out.get(),
      _buf_b.get(), _cur_step_query.get(), M, H, c[13] / Q, Q / c[8], _stream, _tw._is_post_ln,
      nullptr)));
  TAP("encdec_ln_q", _buf_b.get(), mh);
  TAP("res_self", _cur_step_query.get(), mh * sizeof(__half));
}

void QuantDecoder::encdec_attention() {
  const int H = _tw._hidden_size, M = _step_token_num;
  const Layer& w = _layers[_layer_id];
  const float* c = &_dec_clip_max[_layer_id * 19];
  const float Q = _quant_range;

  const size_t mh = (size_t)M * H;
  // Short sources, heads of 64: the q product and the attention are one launch (the same
  // bytes; the context goes to the second part of _buf_a because other workgroups still read
  // the rows of _buf_b).  With taps set the launches below run.
  if (!step_taps.any() && _tw._dim_per_head == 64 &&
      encdec_q_attention_supported(_tw._beam_size, _tw._head_num, H, _batch_seq_len)) {
    int8_t* ctx_q = _buf_a.get() + mh;
    LSH_CALL(encdec_q_attention_f16(
        _buf_b.get(), w.w_encdec_q.get(), w.b_encdec_q.get(),
        _encdec_k.get() + (size_t)_layer_id * _layer_size_encdec_k,
        _encdec_v.get() + (size_t)_layer_id * _layer_size_encdec_k, _p_d_padding_mask, ctx_q,
        Q / c[9], _batch_size, _tw._beam_size, _tw._head_num, _batch_seq_len, H,
        c[2] * c[8] / (c[14] * Q), c[14] / Q, _stream));
    LSH_CALL(gemm_i8_i8o(ctx_q, w.w_encdec_out.get(), _buf_a.get(), M, H, H,
                         c[3] * c[9] / (c[15] * Q), _stream));
    LSH_CALL((residual_bias_ln_i8O<__half, int8_t>(
        _buf_a.get(), w.ffn_ln_scale.get(), w.ffn_ln_bias.get(), w.b_ffn2.get(), _buf_b.get(),
        _cur_step_query.get(), M, H, c[15] / Q, Q / c[10], _stream, _tw._is_post_ln, nullptr)));
    return;
  }
  // q product; its epilogue is ker_arrange_encdec_q_i8I (fp16 q [batch, heads, beam, d])
  if (_tw._dim_per_head % 16 == 0) {
    LSH_CALL(gemm_i8_encdec_q_f16(_buf_b.get(), w.w_encdec_q.get(), w.b_encdec_q.get(),
                                  _query_buf1.get(), M, H, H, _tw._beam_size, _tw._head_num,
                                  c[2] * c[8] / (c[14] * Q), c[14] / Q, _stream));
  } else {
    LSH_CALL(gemm_i8_i8o(_buf_b.get(), w.w_encdec_q.get(), _buf_a.get(), M, H, H,
                         c[2] * c[8] / (c[14] * Q), _stream));
    LSH_CALL(arrange_encdec_q_i8I<__half>(M, H, _stream, _buf_a.get(), w.b_encdec_q.get(),
                                          _query_buf1.get(), _tw._beam_size, _tw._dim_per_head,
                                          _tw._head_num, c[14] / Q));
  }
  TAP("encdec_q", _query_buf1.get(), mh * sizeof(__half));
  TAP("encdec_k", _encdec_k.get() + (size_t)_layer_id * _layer_size_encdec_k,
      (size_t)_batch_token_num * H * sizeof(__half));
  TAP("encdec_v", _encdec_v.get() + (size_t)_layer_id * _layer_size_encdec_k,
      (size_t)_batch_token_num * H * sizeof(__half));
  // scores -> masked softmax -> context -> merge heads + quantise, one kernel
  LSH_CALL(encdec_attention_f16(
      _query_buf1.get(), _encdec_k.get() + (size_t)_layer_id * _layer_size_encdec_k,
      _encdec_v.get() + (size_t)_layer_id * _layer_size_encdec_k, _p_d_padding_mask, nullptr,
      _buf_b.get(), Q / c[9], _batch_size, _tw._beam_size, _tw._head_num, _batch_seq_len,
      _tw._dim_per_head, _stream));
  TAP("encdec_ctx_q", _buf_b.get(), mh);
  LSH_CALL(gemm_i8_i8o(_buf_b.get(), w.w_encdec_out.get(), _buf_a.get(), M, H, H,
                       c[3] * c[9] / (c[15] * Q), _stream));
  TAP("encdec_out_q", _buf_a.get(), mh);
  LSH_CALL((residual_bias_ln_i8O<__half, int8_t>(
      _buf_a.get(), w.ffn_ln_scale.get(), w.ffn_ln_bias.get(), w.b_ffn2.get(), _buf_b.get(),
      _cur_step_query.get(), M, H, c[15] / Q, Q / c[10], _stream, _tw._is_post_ln, nullptr)));
  TAP("ffn_ln_q", _buf_b.get(), mh);
  TAP("res_encdec", _cur_step_query.get(), mh * sizeof(__half));
}

void QuantDecoder::ffn_add_norm() {
  const int H = _tw._hidden_size, I = _tw._inner_size, M = _step_token_num;
  const Layer& w = _layers[_layer_id];
  const float* c = &_dec_clip_max[_layer_id * 19];
  const float Q = _quant_range;

  // FFN1 GEMM with the bias + activation + requantisation in its epilogue
  LSH_CALL(gemm_i8_lut_i8o(_buf_b.get(), w.w_ffn1.get(), _buf_a.get(), w.ffn1_act_lut.get(), M, I,
                           H, c[4] * c[10] / (c[16] * Q), _stream));
  TAP("ffn1_act_q", _buf_a.get(), (size_t)M * I);
  int nparts = 1;
  // a tapped accumulator is one plane (the planes of a split product sum to it exactly)
  const bool tap_acc = step_taps.wants(_layer_id, _cur_step, "ffn2_acc");
  LSH_CALL(gemm_i8_i32o_splitk(_buf_a.get(), w.w_ffn2.get(), _int32_ffn_out_buf.get(), M, H, I,
                               tap_acc ? 1 : gemm_i8_preferred_ksplit(M, H, I), &nparts,
                               _stream));
  TAP("ffn2_acc", _int32_ffn_out_buf.get(), (size_t)M * H * sizeof(int32_t));

  const float dequant_scale =
      _tw._use_gelu ? c[5] * c[11] / (Q * Q) : c[5] * c[11] / (2 * Q * Q);
  const __half *scale_ptr, *bias_ptr, *res_bias_ptr;
  float clip_max;
  if (_layer_id == _tw._n_dec_layer - 1) {
    scale_ptr = _out_ln_scale.get();
    bias_ptr = _out_ln_bias.get();
    res_bias_ptr = nullptr;
    clip_max = _output_ln_clip_max;
  } else {
    const Layer& nx = _layers[_layer_id + 1];
    scale_ptr = nx.self_ln_scale.get();
    bias_ptr = nx.self_ln_bias.get();
    res_bias_ptr = nx.b_self_out.get();
    clip_max = _dec_clip_max[(_layer_id + 1) * 19 + 6];
  }
  LSH_CALL((residual_bias_ln_i8O<__half, int32_t>(
      _int32_ffn_out_buf.get(), scale_ptr, bias_ptr, res_bias_ptr, _buf_a.get(),
      _cur_step_query.get(), M, H, dequant_scale, Q / clip_max, _stream, _tw._is_post_ln,
      w.ffn2_colsum.get(), nparts, (long)M * H)));
  TAP("next_ln_q", _buf_a.get(), (size_t)M * H);
  TAP("res_out", _cur_step_query.get(), (size_t)M * H * sizeof(__half));
}

#undef TAP

// QuantDecoder::sample and ::topk_greedy_search after its first step
// (inference/model/quant_decoder.cc.cu:952-984, 1108-1131): one token per row, in place
void QuantDecoder::sample_tokens() {
  int* alive = _alive_seq[_alive_cur].get();
  CHECK_GPU_ERROR(hipMemsetAsync(_sample_unfinished.get(), 0, sizeof(int), _stream));
  const float dq = _logits_clip_max / _quant_range;
  if (_tw._sampling_method == "topp") {
    LSH_CALL(dec_topp_sample_i8I<__half>(_step_token_num, _cur_step + 1, _tw._max_step, 1, _stream,
                                         _logits.get(), _logit_bias.get(), alive,
                                         _tw._trg_vocab_size, _tw._topp, _sample_unfinished.get(),
                                         _sample_state.get(), _tw._end_id, dq));
  } else {
    const int k = _tw._sampling_method == "topk" ? _tw._topk : 1;
    LSH_CALL(dec_topk_sample_i8I<__half>(_step_token_num, _cur_step + 1, _tw._max_step, 1, _stream,
                                         _logits.get(), _logit_bias.get(), alive,
                                         _tw._trg_vocab_size, k, _sample_unfinished.get(),
                                         _sample_state.get(), _tw._end_id, dq));
  }
  if (_rec_alive && _cur_step < _rec_max_steps)
    CHECK_GPU_ERROR(hipMemcpyAsync(
        _rec_alive + (size_t)_cur_step * _step_token_num * _tw._max_step, alive,
        (size_t)_step_token_num * _tw._max_step * sizeof(int), hipMemcpyDeviceToDevice, _stream));
}

void QuantDecoder::beam_search() {
  int* alive = _alive_seq[_alive_cur].get();
  int* alive_new = _alive_seq[_alive_cur ^ 1].get();
  LSH_CALL(beam_search_step_i8I<__half>(
      _logits.get(), _logit_bias.get(), _alive_seq_probs.get(), _alive_seq_score_own.get(), alive,
      alive_new, _top_score.get(), _top_idx.get(), _parent.get(), _num_finished.get(),
      _logits_clip_max / _quant_range, _tw._trg_vocab_size, _tw._max_step,
      _h_length_norm[_cur_step], _cur_step, _batch_size, _tw._beam_size, _tw._end_id, _stream,
      _topk_part_ws.get(), _topk_part_ws.size()));
  if (_rec_alive && _cur_step < _rec_max_steps)
    CHECK_GPU_ERROR(hipMemcpyAsync(
        _rec_alive + (size_t)_cur_step * _step_token_num * _tw._max_step, alive_new,
        (size_t)_step_token_num * _tw._max_step * sizeof(int), hipMemcpyDeviceToDevice, _stream));

  /* ---refresh cache: k, v for decoder self attention--- (also on a step that turns out to be
   * the last one: the early-stop test reads the finished count after the step) */
  if (_cur_step > 0) {
    LSH_CALL(refresh_cache_by_parent_i8(
        _tw._n_dec_layer, _step_token_num, _stream, _parent.get(),
        _self_k_cache[_cache_cur].get(), _self_v_cache[_cache_cur].get(),
        _self_k_cache[_cache_cur ^ 1].get(), _self_v_cache[_cache_cur ^ 1].get(),
        _layer_size_self_k, _tw._beam_size, _tw._dim_per_head, _tw._head_num, _cur_step,
        _tw._max_step));
  }
}

}  // namespace hip
}  // namespace lightseq
