#include "quant_gpt_encoder.h"

#include "../ls_device.h"

#include <algorithm>

namespace lightseq {
namespace hip {

using namespace lsh;

QuantGptEncoder::QuantGptEncoder(int max_batch_size, const int* p_d_token_id, float* p_d_ppl,
                                 int* p_d_sample_id, const QuantGptWeight& tw, hipStream_t stream)
    : _p_d_token_id(p_d_token_id),
      _p_d_ppl(p_d_ppl),
      _p_d_sample_id(p_d_sample_id),
      _max_batch_size(max_batch_size),
      _tw(tw),
      _stream(stream),
      _src_emb_clip_max(tw._src_emb_clip_max),
      _output_ln_clip_max(tw._output_ln_clip_max),
      _logits_clip_max(tw._logits_clip_max),
      _enc_clip_max(tw._enc_clip_max),
      _atten_scaler(__half2float(__float2half_rn(sqrtf(1.f / (float)std::max(tw._dim_per_head, 1))))),
      _max_batch_dim((long)max_batch_size * tw._max_step * tw._hidden_size) {}

QuantGptEncoder::~QuantGptEncoder() {
  if (_h_unfinished) (void)hipHostFree(_h_unfinished);
}

std::string QuantGptEncoder::check() {
  if (_tw._inner_size & 1) return "violate inner_size % 2 = 0";
  if (_tw._dim_per_head & 1) return "violate dim_per_head % 2 = 0";
  if ((int)_tw.layers.size() != _tw._n_enc_layer)
    return "violate p_d_enc_wei.size() = weight_per_enc_layer * n_enc_layer";
  if ((int)_enc_clip_max.size() != 12 * _tw._n_enc_layer) return "wrong clip_max table size";
  const std::string& m = _tw._sampling_method;
  if (m != "topk" && m != "topp" && m != "ppl")
    return std::string("unsupported sampling_method: ") + m;
  if (m == "topk" && _tw._topk != 1 && _tw._topk != 2 && _tw._topk != 4 && _tw._topk != 8 &&
      _tw._topk != 16 && _tw._topk != 32)
    return "topk argument should be in [1,2,4,8,16,32], the model file has topk = " +
           std::to_string(_tw._topk);
  if (m == "topp" && (!(_tw._topp > 0.f) || _tw._topp > 1.f))
    return "topp must lie in (0, 1], the model file has topp = " + std::to_string(_tw._topp);
  if (_tw._src_vocab_size > (1 << 20)) return "violate vocab_size <= 2^20 (sampling kernels)";
  if (_tw._hidden_size % 16 != 0 || _tw._inner_size % 16 != 0)
    return "violate hidden_size % 16 = 0 and inner_size % 16 = 0 (int8 MFMA GEMM)";
  if (_tw._dim_per_head != 32 && _tw._dim_per_head != 64 && _tw._dim_per_head != 128)
    return "violate dim_per_head in {32, 64, 128} (fused attention kernel)";
  if (_tw._max_step > 4096) return "violate max_step <= 4096";
  if (_tw._eos_id < 0 || _tw._eos_id >= _tw._src_vocab_size)
    return "eos_id outside the vocabulary";
  return "";
}

void QuantGptEncoder::init_buffer() {
  const int H = _tw._hidden_size, I = _tw._inner_size, L = _tw._n_enc_layer;
  const int V = _tw._src_vocab_size;
  const size_t tokens = (size_t)_max_batch_size * _tw._max_step;
  _real_seq_len.alloc(_max_batch_size);
  _ids.alloc(tokens);
  _last_ids.alloc(_max_batch_size);
  _unfinished.alloc(1);
  _sample_state.alloc(2 * (size_t)_max_batch_size);  // 16 bytes per sequence
  set_seed(0);
  CHECK_GPU_ERROR(hipHostMalloc(reinterpret_cast<void**>(&_h_unfinished), sizeof(int)));
  *_h_unfinished = 0;
  _query.alloc((size_t)_max_batch_dim);
  _qkv_buf.alloc((size_t)(3 * _max_batch_dim));
  const size_t wide = tokens * (size_t)std::max(I, 3 * H);
  _buf_a.alloc(wide);
  _buf_b.alloc(wide);
  _buf_q.alloc(wide);
  _hid_last.alloc((size_t)_max_batch_size * H);
  // perplexity needs the logits of every position, sampling only of the last one
  _logits.alloc((_tw._sampling_method == "ppl" ? tokens : (size_t)_max_batch_size) * V);
  // room for the accumulator planes of the split-K second FFN product
  _int32_ffn_out_buf.alloc(std::max(tokens * H * 4, (size_t)64 * H * 8));
  _self_k_cache.alloc((size_t)L * _max_batch_dim);
  _self_v_cache.alloc((size_t)L * _max_batch_dim);
  CHECK_GPU_ERROR(hipMemsetAsync(_self_k_cache.get(), 0, _self_k_cache.size(), _stream));
  CHECK_GPU_ERROR(hipMemsetAsync(_self_v_cache.get(), 0, _self_v_cache.size(), _stream));

  // stored [H, vocab]; one [vocab, H] copy serves the row lookup and the logits GEMM
  _int8_emb = upload_kernel(_tw.token_embedding, H, V, true, _stream);
  _pos_emb = upload_half(_tw.position_embedding, _stream);
  _out_ln_scale = upload_half(_tw.norm_scale, _stream);
  _out_ln_bias = upload_half(_tw.norm_bias, _stream);
  _layers.clear();
  _layers.resize(L);
  for (int l = 0; l < L; ++l) {
    const QuantBertLayerWeight& w = _tw.layers[l];
    Layer& d = _layers[l];
    d.ln1_scale = upload_half(w.multihead_norm_scale, _stream);
    d.ln1_bias = upload_half(w.multihead_norm_bias, _stream);
    d.b_qkv = upload_half(w.multihead_project_bias_qkv, _stream);
    d.b_out = upload_half(w.multihead_project_bias_output, _stream);
    d.ln2_scale = upload_half(w.ffn_norm_scale, _stream);
    d.ln2_bias = upload_half(w.ffn_norm_bias, _stream);
    d.b_ffn1 = upload_half(w.ffn_first_bias, _stream);
    d.b_ffn2 = upload_half(w.ffn_second_bias, _stream);
    d.w_qkv = upload_kernel(w.multihead_project_kernel_qkv, H, 3 * H, true, _stream);
    d.w_out = upload_kernel(w.multihead_project_kernel_output, H, H, true, _stream);
    d.w_ffn1 = upload_kernel(w.ffn_first_kernel, H, I, true, _stream);
    {
      const float* c = &_enc_clip_max[l * 12];
      d.ffn1_act_lut.alloc((size_t)I * 256);
      LSH_CALL(build_act_lut(d.ffn1_act_lut.get(), d.b_ffn1.get(), I, c[10] / _quant_range,
                             _quant_range / c[7], c[7], kActGelu, _stream));
    }
    d.w_ffn2 = upload_kernel(w.ffn_second_kernel, I, H, true, _stream);
  }
  CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
}

// FFN block and the LayerNorm that follows it (:646-776).  `in` holds the int8
// LayerNorm output and receives the next one; `tmp` is scratch of the same size.
// Step taps (debug): name -> what is copied, of the tapped layer at the tapped cached step.
//   ln1_q, self_q, ctx_q, out_q, ln2_q, next_ln_q: int8 [batch, hidden];  act_q: int8 [batch, inner]
//   ffn2_acc: int32 [batch, hidden];  k_cache, v_cache: the layer's int8 caches [batch, heads,
//   max_step, d] after the append;  res_in, res_attn, res_out: the fp16 residual stream [batch,
//   hidden] at the start of the layer, after the first and after the last layer norm
#define TAP(name, ptr, bytes) step_taps.copy(_layer_id, _tap_step, name, ptr, bytes, _stream)

void QuantGptEncoder::ffn_add_norm(int rows, int8_t* in, int8_t* tmp) {
  const int H = _tw._hidden_size, I = _tw._inner_size;
  const Layer& w = _layers[_layer_id];
  const float* c = &_enc_clip_max[_layer_id * 12];
  const float Q = _quant_range;
  LSH_CALL(gemm_i8_lut_i8o(in, w.w_ffn1.get(), tmp, w.ffn1_act_lut.get(), rows, I, H,
                           c[2] * c[6] / (c[10] * Q), _stream));
  TAP("act_q", tmp, (size_t)rows * I);
  int nparts = 1;
  // a tapped accumulator is one plane (the planes of a split product sum to it exactly)
  const bool tap_acc = step_taps.wants(_layer_id, _tap_step, "ffn2_acc");
  LSH_CALL(gemm_i8_i32o_splitk(tmp, w.w_ffn2.get(), _int32_ffn_out_buf.get(), rows, H, I,
                               tap_acc      ? 1
                               : rows <= 64 ? gemm_i8_preferred_ksplit(rows, H, I)
                                            : std::min(4, gemm_i8_preferred_ksplit(rows, H, I)),
                               &nparts, _stream));
  TAP("ffn2_acc", _int32_ffn_out_buf.get(), (size_t)rows * H * sizeof(int32_t));
  const float dequant_scale = c[3] * c[7] / (Q * Q);
  const __half *scale_ptr, *bias_ptr, *res_bias_ptr;
  float clip_max;
  if (_layer_id == _tw._n_enc_layer - 1) {
    scale_ptr = _out_ln_scale.get();
    bias_ptr = _out_ln_bias.get();
    res_bias_ptr = nullptr;
    clip_max = _output_ln_clip_max;
  } else {
    const Layer& nx = _layers[_layer_id + 1];
    scale_ptr = nx.ln1_scale.get();
    bias_ptr = nx.ln1_bias.get();
    res_bias_ptr = nx.b_out.get();
    clip_max = _enc_clip_max[(_layer_id + 1) * 12 + 4];
  }
  LSH_CALL((residual_bias_ln_i8O<__half, int32_t>(
      _int32_ffn_out_buf.get(), scale_ptr, bias_ptr, res_bias_ptr, in, _query.get(), rows, H,
      dequant_scale, Q / clip_max, _stream, false, nullptr, nparts, (long)rows * H)));
  TAP("next_ln_q", in, (size_t)rows * H);
  TAP("res_out", _query.get(), (size_t)rows * H * sizeof(__half));
}

// all prompt positions at once (:253-291 / :299-341); leaves the int8 LayerNorm output of
// the last layer in _buf_a
void QuantGptEncoder::prompt_pass(const int* ids) {
  const int H = _tw._hidden_size, M = _batch_token_num;
  const float Q = _quant_range;
  CHECK_GPU_ERROR(hipMemsetAsync(_real_seq_len.get(), 0, sizeof(int) * _batch_size, _stream));
  LSH_CALL(gpt_embedding_i8I<__half>(_batch_size, _batch_seq_len, H, _stream, _int8_emb.get(),
                                     _pos_emb.get(), ids, _query.get(), _real_seq_len.get(),
                                     _tw._padding_id, 0, _src_emb_clip_max / Q,
                                     _tw._src_vocab_size, _tw._max_step));
  int8_t *a = _buf_a.get(), *b = _buf_b.get();
  __half* qc = _qkv_buf.get();
  __half* kc = qc + _max_batch_dim;
  __half* vd = kc + _max_batch_dim;
  const bool on_codes =
      gpt_prefill_i8_enabled() && H % 128 == 0 &&
      gpt_prefill_i8_supported(_batch_seq_len, _tw._head_num, _tw._dim_per_head);
  for (_layer_id = 0; _layer_id < _tw._n_enc_layer; _layer_id++) {
    const Layer& w = _layers[_layer_id];
    const float* c = &_enc_clip_max[_layer_id * 12];
    if (_layer_id == 0)
      LSH_CALL(norm_layer_resual_i8O<__half>(M, H, _stream, _query.get(), a, w.ln1_scale.get(),
                                             w.ln1_bias.get(), w.b_out.get(), Q / c[4], false));
    LSH_CALL(gemm_i8_i8o(a, w.w_qkv.get(), b, M, 3 * H, H, c[0] * c[4] / (c[8] * Q), _stream));
    int8_t* k_cache = _self_k_cache.get() + (size_t)_layer_id * _max_batch_dim;
    int8_t* v_cache = _self_v_cache.get() + (size_t)_layer_id * _max_batch_dim;
    if (on_codes) {
      // int8 end to end: q codes and the caches are all the arrange stage writes, and the
      // attention reads them
      int8_t* q8 = reinterpret_cast<int8_t*>(qc);
      LSH_CALL(gpt_arrange_qkv_prefill_i8(M, H, _stream, b, w.b_qkv.get(), q8, k_cache, v_cache,
                                          _batch_seq_len, _tw._dim_per_head, _tw._head_num,
                                          _tw._max_step, c[8] / Q, Q / c[11]));
      LSH_CALL(gpt_prefill_attention_i8(q8, k_cache, v_cache, _real_seq_len.get(), a, Q / c[5],
                                        c[11] / Q, Q / c[11], _batch_size, _batch_seq_len,
                                        _tw._head_num, _tw._dim_per_head, _tw._max_step, _stream));
    } else {
      LSH_CALL(gpt_arrange_qkv_prefill_f16(M, H, _stream, b, w.b_qkv.get(), qc, kc, vd, k_cache,
                                           v_cache, _batch_seq_len, _tw._dim_per_head,
                                           _tw._head_num, _tw._max_step, c[8] / Q, Q / c[11]));
      LSH_CALL(gpt_prefill_attention_f16(qc, kc, vd, _real_seq_len.get(), nullptr, a, Q / c[5],
                                         c[11] / Q, _batch_size, _batch_seq_len, _tw._head_num,
                                         _tw._dim_per_head, _stream));
    }
    LSH_CALL(gemm_i8_i8o(a, w.w_out.get(), b, M, H, H, c[1] * c[5] / (c[9] * Q), _stream));
    LSH_CALL((residual_bias_ln_i8O<__half, int8_t>(b, w.ln2_scale.get(), w.ln2_bias.get(),
                                                   w.b_ffn2.get(), a, _query.get(), M, H,
                                                   c[9] / Q, Q / c[6], _stream, false, nullptr)));
    ffn_add_norm(M, a, b);
  }
}

// one cached step for the tokens in _last_ids at position _batch_seq_len - 1 (:363-377);
// returns the buffer that holds the int8 LayerNorm output of the last layer [batch, hidden]
const int8_t* QuantGptEncoder::step_pass() {
  LnFewRowsScope few_rows;  // every step of every batch size: layer norms by the row kernel
  const int H = _tw._hidden_size, B = _batch_size;
  const float Q = _quant_range;
  int8_t *a = _buf_a.get(), *b = _buf_b.get();
  _tap_step = _steps_run;
  // the step's embedding and the first layer norm are one launch where the row kernel covers
  // the width (the same bytes); with taps set the two launches run
  const bool emb_ln_fused = !step_taps.any() && H % 4 == 0 && H <= 1024 && _tw._n_enc_layer > 0;
  if (emb_ln_fused) {
    const Layer& w0 = _layers[0];
    LSH_CALL(gpt_emb_step_norm_layer_i8O<__half>(
        _int8_emb.get(), _pos_emb.get(), _last_ids.get(), _query.get(), a, w0.ln1_scale.get(),
        w0.ln1_bias.get(), w0.b_out.get(), _real_seq_len.get(), _unfinished.get(), B, H,
        _tw._src_vocab_size, _tw._padding_id, _batch_seq_len - 1, _tw._max_step,
        _src_emb_clip_max / Q, Q / _enc_clip_max[4], false, _stream));
  } else {
    LSH_CALL(gpt_embedding_i8I<__half>(B, 1, H, _stream, _int8_emb.get(), _pos_emb.get(),
                                       _last_ids.get(), _query.get(), _real_seq_len.get(),
                                       _tw._padding_id, _batch_seq_len - 1, _src_emb_clip_max / Q,
                                       _tw._src_vocab_size, _tw._max_step, _unfinished.get()));
  }
  const size_t bh = (size_t)B * H;
  for (_layer_id = 0; _layer_id < _tw._n_enc_layer; _layer_id++) {
    const Layer& w = _layers[_layer_id];
    const float* c = &_enc_clip_max[_layer_id * 12];
    int8_t* k_cache = _self_k_cache.get() + (size_t)_layer_id * _max_batch_dim;
    int8_t* v_cache = _self_v_cache.get() + (size_t)_layer_id * _max_batch_dim;
    if (_layer_id == 0 && !emb_ln_fused)
      LSH_CALL(norm_layer_resual_i8O<__half>(B, H, _stream, _query.get(), a, w.ln1_scale.get(),
                                             w.ln1_bias.get(), w.b_out.get(), Q / c[4], false));
    TAP("ln1_q", a, bh);
    TAP("res_in", _query.get(), bh * sizeof(__half));
    // With taps set the two launches run, so that q and the caches are copied before the
    // attention as the tap names promise.
    if (!step_taps.any() && decself_qkv_attention_enabled() && _tw._dim_per_head == 64 &&
        decself_qkv_attention_supported(B, H, _tw._head_num, _tw._max_step)) {
      LSH_CALL(decself_qkv_attention_i8(a, w.w_qkv.get(), w.b_qkv.get(), _buf_q.get(), k_cache,
                                        v_cache, b, B, H, _tw._head_num, _tw._max_step,
                                        _batch_seq_len - 1, c[0] * c[4] / (c[8] * Q), c[8] / Q,
                                        Q / c[11], _atten_scaler, c[11] / Q, Q / c[5], _stream));
    } else {
    // QKV product; its epilogue is ker_arrange_decself_qkv_i8I_i8O: q -> _buf_q, k / v appended
    // to the caches at the token's position
    if (_tw._dim_per_head % 16 == 0) {
      LSH_CALL(gemm_i8_decself_qkv_i8o(a, w.w_qkv.get(), w.b_qkv.get(), _buf_q.get(), k_cache,
                                       v_cache, B, H, H, _tw._head_num, _tw._max_step,
                                       _batch_seq_len - 1, c[0] * c[4] / (c[8] * Q), c[8] / Q,
                                       Q / c[11], _stream));
    } else {
      LSH_CALL(gemm_i8_i8o(a, w.w_qkv.get(), b, B, 3 * H, H, c[0] * c[4] / (c[8] * Q), _stream));
      LSH_CALL(arrange_decself_qkv_i8I_i8O<__half>(B, H, _stream, b, w.b_qkv.get(), _buf_q.get(),
                                                   k_cache, v_cache, _tw._head_num,
                                                   _tw._dim_per_head, _tw._max_step,
                                                   _batch_seq_len - 1, c[8] / Q, Q / c[11]));
    }
    TAP("self_q", _buf_q.get(), bh);
    TAP("k_cache", k_cache, bh * _tw._max_step);
    TAP("v_cache", v_cache, bh * _tw._max_step);
    LSH_CALL(decself_attention_i8(_buf_q.get(), k_cache, v_cache, b, B * _tw._head_num,
                                  _batch_seq_len,
                                  _tw._max_step, _tw._head_num, _tw._dim_per_head, _atten_scaler,
                                  c[11] / Q, Q / c[5], _stream));
    }
    TAP("ctx_q", b, bh);
    LSH_CALL(gemm_i8_i8o(b, w.w_out.get(), a, B, H, H, c[1] * c[5] / (c[9] * Q), _stream));
    TAP("out_q", a, bh);
    LSH_CALL((residual_bias_ln_i8O<__half, int8_t>(a, w.ln2_scale.get(), w.ln2_bias.get(),
                                                   w.b_ffn2.get(), b, _query.get(), B, H,
                                                   c[9] / Q, Q / c[6], _stream, false, nullptr)));
    TAP("ln2_q", b, bh);
    TAP("res_attn", _query.get(), bh * sizeof(__half));
    ffn_add_norm(B, b, a);
    std::swap(a, b);  // `a` names the buffer holding the layer's int8 LayerNorm output
  }
  _tap_step = -2;
  return a;
}

#undef TAP

// logits of the last position + greedy choice, enqueued only (:399-487)
void QuantGptEncoder::enqueue_sampling(const int8_t* hidden, bool clear_flag) {
  const int H = _tw._hidden_size, V = _tw._src_vocab_size, B = _batch_size;
  LSH_CALL(gemm_i8_i8o(hidden, _int8_emb.get(), _logits.get(), B, V, H,
                       _output_ln_clip_max * _src_emb_clip_max / (_logits_clip_max * _quant_range),
                       _stream));
  if (_rec_logits && _steps_run < _rec_max_steps)
    CHECK_GPU_ERROR(hipMemcpyAsync(_rec_logits + (size_t)_steps_run * B * V, _logits.get(),
                                   (size_t)B * V, hipMemcpyDeviceToDevice, _stream));
  // (after a cached step the flag was cleared by the step's embedding launch)
  if (clear_flag) LSH_CALL(fill_i32(_unfinished.get(), 0, 1, _stream));
  const bool topp = _tw._sampling_method == "topp";
  if (!topp && _tw._topk == 1) {
    LSH_CALL(gpt_greedy_step(_logits.get(), _ids.get(), _last_ids.get(), V, _tw._max_step,
                             _batch_seq_len, B, _unfinished.get(), _tw._eos_id, _stream));
  } else {
    // ker_topk_sample_i8I<k> / ker_topp_sample_i8I (:405-430, :448-473)
    LSH_CALL(gpt_sample_step(_logits.get(), _ids.get(), _last_ids.get(), V, _tw._max_step,
                             _batch_seq_len, B, _unfinished.get(), _tw._eos_id,
                             topp ? 0 : _tw._topk, _tw._topp, _logits_clip_max / _quant_range,
                             _sample_state.get(), _stream));
  }
}

// Restart the generator states of the random-sampling steps: sequence i draws from (seed, i).
void QuantGptEncoder::set_seed(unsigned long long seed) {
  LSH_CALL(sample_state_setup(_sample_state.get(), _max_batch_size, seed, _stream));
}

// host side of a sampled token: counters and the unfinished flag (one word back from the device)
int QuantGptEncoder::finish_token() {
  const int B = _batch_size;
  const bool first = _steps_run == 0;
  ++_steps_run;
  _batch_seq_len++;
  _batch_token_num += B;
  if (_is_benchmark && !first) return 1;  // nothing stops a benchmark run but the length
  CHECK_GPU_ERROR(hipMemcpyAsync(_h_unfinished, _unfinished.get(), sizeof(int),
                                 hipMemcpyDeviceToHost, _stream));
  CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
  return *_h_unfinished;
}

int QuantGptEncoder::run_one_sample(int batch_size, int batch_seq_len) {
  if (batch_size > _max_batch_size)
    throw std::runtime_error("batch size of input greater than max_batch_size");
  if (batch_seq_len > _tw._max_step)
    throw std::runtime_error("seq len of input greater than max_step");
  if (batch_size <= 0 || batch_seq_len <= 0) throw std::runtime_error("empty input");
  if (_tw._sampling_method == "ppl")
    throw std::runtime_error("this model file is configured for perplexity, not sampling");
  _batch_size = batch_size;
  _batch_seq_len = batch_seq_len;
  _batch_token_num = batch_size * batch_seq_len;
  _batch_max_seq_len = std::min(_tw._max_step, batch_seq_len + _tw._extra_decode_length);
  _steps_run = 0;
  const int H = _tw._hidden_size;

  _phases.mark(0, _stream);
  // ids [batch, max_step] <- prompt
  CHECK_GPU_ERROR(hipMemcpy2DAsync(_ids.get(), sizeof(int) * _tw._max_step, _p_d_token_id,
                                   sizeof(int) * batch_seq_len, sizeof(int) * batch_seq_len,
                                   batch_size, hipMemcpyDeviceToDevice, _stream));
  prompt_pass(_p_d_token_id);
  // hidden states of the last prompt position of every sequence
  CHECK_GPU_ERROR(hipMemcpy2DAsync(_hid_last.get(), H,
                                   _buf_a.get() + (size_t)(batch_seq_len - 1) * H,
                                   (size_t)batch_seq_len * H, H, batch_size,
                                   hipMemcpyDeviceToDevice, _stream));
  int loop_steps = 0;
  if (_batch_seq_len < _tw._max_step) {
    // (:347-353) after the prompt pass the run ends when nothing is unfinished
    enqueue_sampling(_hid_last.get(), true);
    const bool go_on = !(finish_token() == 0 || _batch_seq_len >= _batch_max_seq_len);
    _phases.mark(1, _stream);
    if (go_on) {
      while (_batch_seq_len < _batch_max_seq_len) {
        ++loop_steps;
        // the launches of a step depend on the batch size and the position only
        const uint64_t key = ((uint64_t)_batch_size << 32) | (uint32_t)_batch_seq_len;
        _graphs.run(key, _stream, _use_graphs && !_rec_logits && !step_taps.any(),
                    [&] { enqueue_sampling(step_pass(), false); });
        int unfinished = finish_token();
        if (!unfinished && !_is_benchmark) break;
      }
    }
  } else {
    _phases.mark(1, _stream);
  }
  _phases.mark(2, _stream);
  _phases.set_loop_steps(loop_steps);
  CHECK_GPU_ERROR(hipMemcpy2DAsync(_p_d_sample_id, sizeof(int) * _batch_seq_len, _ids.get(),
                                   sizeof(int) * _tw._max_step, sizeof(int) * _batch_seq_len,
                                   batch_size, hipMemcpyDeviceToDevice, _stream));
  CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
  return _batch_seq_len;
}

void QuantGptEncoder::run_one_infer(int batch_size, int batch_seq_len) {
  if (batch_size > _max_batch_size)
    throw std::runtime_error("batch size of input greater than max_batch_size");
  if (batch_seq_len > _tw._max_step)
    throw std::runtime_error("seq len of input greater than max_step");
  if (batch_size <= 0 || batch_seq_len <= 0) throw std::runtime_error("empty input");
  if (_tw._sampling_method != "ppl")
    throw std::runtime_error("this model file is configured for sampling, not perplexity");
  _batch_size = batch_size;
  _batch_seq_len = batch_seq_len;
  _batch_token_num = batch_size * batch_seq_len;
  const int H = _tw._hidden_size, V = _tw._src_vocab_size;
  CHECK_GPU_ERROR(hipMemsetAsync(_p_d_ppl, 0, sizeof(float) * batch_size, _stream));
  prompt_pass(_p_d_token_id);
  /* compute_ppl (:781-797) */
  LSH_CALL(gemm_i8_i8o(_buf_a.get(), _int8_emb.get(), _logits.get(), _batch_token_num, V, H,
                       _output_ln_clip_max * _src_emb_clip_max / (_logits_clip_max * _quant_range),
                       _stream));
  // the FFN2 accumulator buffer (tokens * hidden int32, idle by now) holds the per-position terms
  LSH_CALL(ppl_i8I(batch_size, batch_seq_len, _stream, _logits.get(), _p_d_token_id,
                   _real_seq_len.get(), _p_d_ppl, V, _logits_clip_max / _quant_range,
                   reinterpret_cast<float*>(_int32_ffn_out_buf.get())));
}

}  // namespace hip
}  // namespace lightseq
