#include "quant_bert_encoder.h"

#include "../ls_device.h"

#include <algorithm>

namespace lightseq {
namespace hip {

// polls (about a microsecond each) after which a wait inside the feed-forward segment gives up
static const int kSegmentSpinLimit = 1 << 15;

using namespace lsh;

QuantBertEncoder::QuantBertEncoder(int max_batch_size, const int* p_d_token_id,
                                   int* p_d_padding_mask, __half* p_d_output,
                                   const QuantBertWeight& tw, hipStream_t stream)
    : _p_d_token_id(p_d_token_id),
      _p_d_padding_mask(p_d_padding_mask),
      _p_d_output(p_d_output),
      _max_batch_size(max_batch_size),
      _tw(tw),
      _stream(stream),
      _src_emb_clip_max(tw._src_emb_clip_max),
      _enc_clip_max(tw._enc_clip_max),
      _max_batch_dim((long)max_batch_size * tw._max_step * tw._hidden_size) {}

std::string QuantBertEncoder::check() {
  if (_tw._inner_size & 1) return "violate inner_size % 2 = 0";
  if (_tw._dim_per_head & 1) return "violate dim_per_head % 2 = 0";
  if (_tw._multilg_type != 0) return "multilingual models are not supported";
  if ((int)_tw.layers.size() != _tw._n_enc_layer)
    return "violate p_d_enc_wei.size() = weight_per_enc_layer * n_enc_layer";
  if ((int)_enc_clip_max.size() != _tw._clip_stride * _tw._n_enc_layer)
    return "wrong clip_max table size";
  if (_tw._hidden_size % 16 != 0 || _tw._inner_size % 16 != 0)
    return "violate hidden_size % 16 = 0 and inner_size % 16 = 0 (int8 MFMA GEMM)";
  if (_tw._dim_per_head != 32 && _tw._dim_per_head != 64 && _tw._dim_per_head != 128)
    return "violate dim_per_head in {32, 64, 128} (fused attention kernel)";
  if (_tw._max_step > 1024) return "violate max_step <= 1024";
  return "";
}

void QuantBertEncoder::init_buffer() {
  const int H = _tw._hidden_size, I = _tw._inner_size;
  const long tokens = (long)_max_batch_size * _tw._max_step;
  _qkv_buf.alloc((size_t)(3 * _max_batch_dim));
  const size_t wide = (size_t)tokens * std::max(I, 3 * H);
  _int8_ffn_in_buf.alloc(wide);
  _int8_ffn_out_buf.alloc(wide);
  // room for the accumulator planes of a split-K second FFN product (up to 4 at encoder
  // sizes, up to 8 for the few rows of a decode step)
  _int32_ffn_out_buf.alloc(std::max((size_t)tokens * H * 4, (size_t)64 * H * 8));
  _qa_plan.alloc((size_t)_max_batch_size * _tw._head_num);
  _seg_sync.alloc(ffn_segment_sync_words());
  CHECK_GPU_ERROR(hipMemsetAsync(_seg_sync.get(), 0, _seg_sync.size() * sizeof(unsigned), _stream));
  CHECK_GPU_ERROR(hipHostMalloc(reinterpret_cast<void**>(&_h_seg_error), sizeof(unsigned)));
  *_h_seg_error = 0;

  _int8_emb = upload_kernel(_tw.token_embedding, _tw._src_vocab_size, H, false, _stream);
  _pos_emb = upload_half(_tw.position_embedding, _stream);
  _final_ln_scale = upload_half(_tw.norm_scale, _stream);
  _final_ln_bias = upload_half(_tw.norm_bias, _stream);

  _layers.clear();
  _layers.resize(_tw._n_enc_layer);
  for (int l = 0; l < _tw._n_enc_layer; ++l) {
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
    if (gemm_ln_fused_supported(H, H)) {
      d.w_out_tiled.alloc((size_t)H * H);
      LSH_CALL(tile_weight_16x64(d.w_out.get(), d.w_out_tiled.get(), H, H, _stream));
    }
    d.w_ffn1 = upload_kernel(w.ffn_first_kernel, H, I, true, _stream);
    d.w_ffn2 = upload_kernel(w.ffn_second_kernel, I, H, true, _stream);
    {
      // table of the FFN1 epilogue (dequantise, bias, activation, requantise) per output code
      const float* c = &_enc_clip_max[l * _tw._clip_stride];
      d.ffn1_act_lut.alloc((size_t)I * 256);
      LSH_CALL(build_act_lut(d.ffn1_act_lut.get(), d.b_ffn1.get(), I, c[10] / _quant_range,
                             _quant_range / c[7], c[7],
                             _tw._use_gelu ? kActGelu : kActReluNarrow, _stream));
    }
    if (!_tw._use_gelu) {
      // ReLU offset trick: colsum of the fp16-rounded dequantised FFN2 weight times
      // clip/2 (quant_bert_encoder.cc.cu:156-175)
      const size_t n = w.ffn_second_kernel.size();
      DeviceBuffer<uint8_t> raw(n);
      raw.upload(w.ffn_second_kernel.data(), n, _stream);
      DeviceBuffer<__half> deq(n);
      LSH_CALL(stored_u8_dequant<__half>(raw.get(), deq.get(), (long)n, _enc_clip_max[l * _tw._clip_stride + 3],
                                         _stream));
      d.ffn2_colsum.alloc(H);
      LSH_CALL(scaled_colsum<__half>(deq.get(), d.ffn2_colsum.get(), I, H,
                                     _enc_clip_max[l * _tw._clip_stride + 7] / 2, _stream));
      CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
    }
  }
}

void QuantBertEncoder::set_profiling(bool on) {
  _profiling = on;
  if (on && _profile.empty()) {
    _profile.resize(4);
    const char* names[4] = {"qkv", "attn_out", "ffn1", "ffn2"};
    for (int i = 0; i < 4; ++i) _profile[i].site = names[i];
  }
}

void QuantBertEncoder::reset_profile() {
  for (auto& p : _profile) { p.launches = 0; p.total_ms = 0.0; }
}

void QuantBertEncoder::prof_begin(int site, int m, int n, int k, const char* epilogue) {
  if (!_profiling) return;
  const bool fused_ln = std::string(epilogue) == "fused_ln";
  const bool fused_qa = std::string(epilogue) == "fused_qkv_attn";
  const bool segment = std::string(epilogue) == "ffn_segment";
  SiteProfile& p = _profile[site];
  if (p.m != m || p.n != n || p.k != k || p.kernel.empty() || p.route != epilogue) {
    p.m = m; p.n = n; p.k = k;
    p.route = epilogue;
    p.kernel = fused_ln   ? "gemm_ln_rows16_kernel"
               : fused_qa ? "qkv_attn_kernel"
               : segment  ? "ffn_segment_kernel"
                          : gemm_i8_kernel_name(m, n, k, epilogue);
  }
  Pending pe;
  pe.site = site;
  for (hipEvent_t* e : {&pe.e0, &pe.e1}) {
    if (_event_pool.empty()) {
      CHECK_GPU_ERROR(hipEventCreate(e));
    } else {
      *e = _event_pool.back();
      _event_pool.pop_back();
    }
  }
  // the launcher records the kernel's own begin / end timestamps into the events
  if (fused_ln) gemm_ln_time_next_launch(pe.e0, pe.e1);
  else if (fused_qa) qkv_attention_time_next_launch(pe.e0, pe.e1);
  else if (segment) ffn_segment_time_next_launch(pe.e0, pe.e1);
  else gemm_i8_time_next_launch(pe.e0, pe.e1);
  _pending.push_back(pe);
}

void QuantBertEncoder::collect_profile() {
  for (Pending& pe : _pending) {
    float ms = 0.f;
    CHECK_GPU_ERROR(hipEventElapsedTime(&ms, pe.e0, pe.e1));
    _profile[pe.site].launches += 1;
    _profile[pe.site].total_ms += ms;
    _event_pool.push_back(pe.e0);
    _event_pool.push_back(pe.e1);
  }
  _pending.clear();
}

QuantBertEncoder::~QuantBertEncoder() {
  ffn_segment_release(this);
  if (_h_seg_error) (void)hipHostFree(_h_seg_error);
}

bool QuantBertEncoder::finish_infer() {
  if (!_seg_active) return false;
  _seg_active = false;
  ffn_segment_release(this);
  if (*_h_seg_error == 0) return false;
  // a wait inside the segment kernel gave up: its outputs are undefined.  Clear the counters,
  // leave that route, and let the caller run the batch again on the three launches.
  CHECK_GPU_ERROR(hipMemsetAsync(_seg_sync.get(), 0, _seg_sync.size() * sizeof(unsigned), _stream));
  CHECK_GPU_ERROR(hipStreamSynchronize(_stream));
  _seg_launches = 0;
  *_h_seg_error = 0;
  _seg_off = true;
  return true;
}

void QuantBertEncoder::tap(int8_t* dst, const int8_t* src, size_t n) {
  if (dst && taps.tap_layer == _layer_id)
    CHECK_GPU_ERROR(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, _stream));
}

void QuantBertEncoder::run_one_infer(int batch_size, int batch_seq_len) {
  if (batch_size > _max_batch_size)
    throw std::runtime_error("batch size of input greater than max_batch_size");
  if (batch_seq_len > _tw._max_step)
    throw std::runtime_error("seq len of input greater than max_step");
  if (batch_size <= 0 || batch_seq_len <= 0) throw std::runtime_error("empty input");
  _batch_size = batch_size;
  _batch_seq_len = batch_seq_len;
  _batch_token_num = batch_size * batch_seq_len;

  LSH_CALL(enc_emb_i8I<__half>(_int8_emb.get(), _pos_emb.get(), _p_d_token_id, _p_d_output,
                               _p_d_padding_mask, _tw._padding_id, batch_size, batch_seq_len,
                               _tw._hidden_size, _stream, _src_emb_clip_max / _quant_range,
                               _tw._scale_embedding, _tw._src_vocab_size));
  // one plan for the fused QKV + attention launches of all layers: the padding mask is theirs all
  _qa_plan_cur = nullptr;
  if (_fuse && qkv_attention_plan_enabled() &&
      qkv_attention_fused_supported(batch_size, batch_seq_len, _tw._head_num, _tw._dim_per_head) &&
      qkv_attention_plan_supported(batch_size, batch_seq_len, _tw._head_num)) {
    LSH_CALL(qkv_attention_plan(_p_d_padding_mask, _qa_plan.get(), batch_size, batch_seq_len,
                                _tw._head_num, _stream));
    _qa_plan_cur = _qa_plan.get();
  }
  _seg_active = _fuse && !_seg_off && ffn_segment_enabled() && _seg_sync.get() != nullptr &&
                ffn_segment_supported(_batch_token_num, _tw._hidden_size, _tw._inner_size) &&
                ffn_segment_claim(this);
  for (_layer_id = 0; _layer_id < _tw._n_enc_layer; _layer_id++) {
    self_attention();
    ffn_add_norm();
  }
  if (_seg_active)
    CHECK_GPU_ERROR(hipMemcpyAsync(_h_seg_error, _seg_sync.get() + _seg_sync.size() - 1,
                                   sizeof(unsigned), hipMemcpyDeviceToHost, _stream));
}

void QuantBertEncoder::self_attention() {
  const int H = _tw._hidden_size, M = _batch_token_num;
  const Layer& w = _layers[_layer_id];
  const float* c = &_enc_clip_max[_layer_id * _tw._clip_stride];
  const float Q = _quant_range;

  if (_layer_id == 0) {
    LSH_CALL(norm_layer_resual_i8O<__half>(M, H, _stream, _p_d_output, _int8_ffn_in_buf.get(),
                                           w.ln1_scale.get(), w.ln1_bias.get(), w.b_out.get(),
                                           Q / c[4], _tw._is_post_ln));
  }
  tap(taps.ln1_q, _int8_ffn_in_buf.get(), (size_t)M * H);

  // qkv = ori_q * qkv_wei -> int8 codes [M, 3H] -> fp16 q, k, v -> attention -> int8 context.
  // Three routes with the same bits: (a) one kernel per (sequence, head) that keeps codes and
  // q, k, v on the compute unit (heads of 64, at most 128 tokens, codes not tapped); (b) the
  // GEMM, then an attention kernel that dequantises the codes as it stages q, k, v; (c) the
  // GEMM, the arrange kernel writing fp16 q, k, v [B, h, S, d], the attention on those.
  const long mbd = (long)M * H;
  const int dph = _tw._dim_per_head;
  const bool tap_qkv = taps.qkv_q && taps.tap_layer == _layer_id;
  if (_fuse && !tap_qkv &&
      qkv_attention_fused_supported(_batch_size, _batch_seq_len, _tw._head_num, dph)) {
    prof_begin(0, M, 3 * H, H, "fused_qkv_attn");
    // reads _int8_ffn_in_buf and must not overwrite it: the context goes to _int8_ffn_out_buf
    // and the two buffers swap roles
    LSH_CALL(qkv_attention_i8(_int8_ffn_in_buf.get(), w.w_qkv.get(), w.b_qkv.get(),
                              _p_d_padding_mask, _int8_ffn_out_buf.get(), c[0] * c[4] / (c[8] * Q),
                              c[8] / Q, Q / c[5], _batch_size, _batch_seq_len, _tw._head_num, dph,
                              _stream, _qa_plan_cur));
    std::swap(_int8_ffn_in_buf, _int8_ffn_out_buf);
  } else {
    prof_begin(0, M, 3 * H, H, "EpiI8");
    LSH_CALL(gemm_i8_i8o(_int8_ffn_in_buf.get(), w.w_qkv.get(), _int8_ffn_out_buf.get(), M, 3 * H,
                         H, c[0] * c[4] / (c[8] * Q), _stream));
    tap(taps.qkv_q, _int8_ffn_out_buf.get(), (size_t)M * 3 * H);
    if (_fuse && (dph == 32 || dph == 64 || dph == 128)) {
      // scores -> masked softmax -> context -> merge heads + quantise, one kernel
      LSH_CALL(encself_attention_i8qkv(_int8_ffn_out_buf.get(), w.b_qkv.get(), c[8] / Q,
                                       _p_d_padding_mask, nullptr, _int8_ffn_in_buf.get(),
                                       Q / c[5], _batch_size, _batch_seq_len, _tw._head_num, dph,
                                       _stream));
    } else {
      LSH_CALL(arrange_encself_qkv_i8I<__half>(M, H, _stream, _int8_ffn_out_buf.get(),
                                               w.b_qkv.get(), _qkv_buf.get(), mbd, _batch_seq_len,
                                               dph, _tw._head_num, c[8] / Q));
      LSH_CALL(encself_attention_f16(_qkv_buf.get(), _qkv_buf.get() + mbd,
                                     _qkv_buf.get() + 2 * mbd, _p_d_padding_mask, nullptr,
                                     _int8_ffn_in_buf.get(), Q / c[5], _batch_size, _batch_seq_len,
                                     _tw._head_num, dph, _stream));
    }
  }
  tap(taps.ctx_q, _int8_ffn_in_buf.get(), (size_t)M * H);

  const bool tap_out = (taps.out_q || taps.res_attn) && taps.tap_layer == _layer_id;
  if (_fuse && !tap_out && w.w_out_tiled.get() != nullptr) {
    // out-projection + dequant + residual + LayerNorm + quant in one kernel: the int8 product
    // never reaches memory.  Same bytes as the pair below; reads _int8_ffn_in_buf (context codes)
    // and must not overwrite it, so the LayerNorm output goes to _int8_ffn_out_buf and the two
    // buffers swap roles.
    prof_begin(1, M, H, H, "fused_ln");
    LSH_CALL(gemm_i8_residual_ln_i8O<__half>(
        _int8_ffn_in_buf.get(), w.w_out_tiled.get(), c[1] * c[5] / (c[9] * Q), w.ln2_scale.get(),
        w.ln2_bias.get(), w.b_ffn2.get(), _int8_ffn_out_buf.get(), _p_d_output, M, H, H, c[9] / Q,
        Q / c[6], _stream, _tw._is_post_ln));
    std::swap(_int8_ffn_in_buf, _int8_ffn_out_buf);
  } else {
    prof_begin(1, M, H, H, "EpiI8");
    LSH_CALL(gemm_i8_i8o(_int8_ffn_in_buf.get(), w.w_out.get(), _int8_ffn_out_buf.get(), M, H, H,
                         c[1] * c[5] / (c[9] * Q), _stream));
    tap(taps.out_q, _int8_ffn_out_buf.get(), (size_t)M * H);

    if (taps.res_attn && taps.tap_layer == _layer_id)
      CHECK_GPU_ERROR(hipMemcpyAsync(taps.res_attn, _p_d_output, (size_t)M * H * sizeof(__half),
                                     hipMemcpyDeviceToDevice, _stream));
    LSH_CALL((residual_bias_ln_i8O<__half, int8_t>(
        _int8_ffn_out_buf.get(), w.ln2_scale.get(), w.ln2_bias.get(), w.b_ffn2.get(),
        _int8_ffn_in_buf.get(), _p_d_output, M, H, c[9] / Q, Q / c[6], _stream, _tw._is_post_ln,
        nullptr)));
  }
  tap(taps.ln2_q, _int8_ffn_in_buf.get(), (size_t)M * H);
}

void QuantBertEncoder::ffn_add_norm() {
  const int H = _tw._hidden_size, I = _tw._inner_size, M = _batch_token_num;
  const Layer& w = _layers[_layer_id];
  const float* c = &_enc_clip_max[_layer_id * _tw._clip_stride];
  const float Q = _quant_range;

  const float dequant_scale =
      _tw._use_gelu ? c[3] * c[7] / (Q * Q) : c[3] * c[7] / (2 * Q * Q);
  const __half* colsum = w.ffn2_colsum.get();  // nullptr for GELU models
  const bool last = _layer_id == _tw._n_enc_layer - 1;
  const bool tapped = taps.tap_layer == _layer_id && (taps.ffn1_q || taps.ffn2_acc || taps.res_ffn);
  if (_seg_active && !tapped) {
    // FFN1 + table, FFN2 and the layer norm in one launch (the bytes of the three launches
    // below).  Reads _int8_ffn_in_buf, leaves the activation codes in _int8_ffn_out_buf and the
    // next layer's input codes in _int8_ffn_in_buf.
    prof_begin(2, M, I, H, "ffn_segment");
    const Layer* nx = last ? nullptr : &_layers[_layer_id + 1];
    const float clip_next = last ? 1.f : _enc_clip_max[(_layer_id + 1) * _tw._clip_stride + 4];
    // the last phase writes the next layer's codes over the rows the first phase read: rows
    // belong to one XCD, whose workgroups have all left the first phase by then
    LSH_CALL(ffn_segment_i8(
        _int8_ffn_in_buf.get(), w.w_ffn1.get(), w.ffn1_act_lut.get(), c[2] * c[6] / (c[10] * Q),
        _int8_ffn_out_buf.get(), w.w_ffn2.get(), _int32_ffn_out_buf.get(), _p_d_output,
        last ? _p_d_output : nullptr, last ? nullptr : _int8_ffn_in_buf.get(),
        last ? _final_ln_scale.get() : nx->ln1_scale.get(),
        last ? _final_ln_bias.get() : nx->ln1_bias.get(), last ? nullptr : nx->b_out.get(), colsum,
        M, H, I, dequant_scale, last ? 0.f : Q / clip_next, _tw._is_post_ln, last, _seg_sync.get(),
        &_seg_launches, kSegmentSpinLimit, _stream));
    tap(taps.act_q, _int8_ffn_out_buf.get(), (size_t)M * I);
    return;
  }

  // FFN1 -> int8 code -> dequant + bias + activation + requant.  Fused into the GEMM
  // epilogue unless the int8 GEMM output is tapped; both routes give the same bits.
  // The fused GEMM reads _int8_ffn_in_buf and must not overwrite it: it writes to
  // _int8_ffn_out_buf and the two buffers swap roles for the rest of the layer.
  const bool tap_ffn1 = taps.ffn1_q && taps.tap_layer == _layer_id;
  const int act = _tw._use_gelu ? kActGelu : kActReluNarrow;
  int8_t* act_buf = _int8_ffn_in_buf.get();
  if (_fuse && !tap_ffn1) {
    (void)act;
    prof_begin(2, M, I, H, "EpiLutI8");
    LSH_CALL(gemm_i8_lut_i8o(_int8_ffn_in_buf.get(), w.w_ffn1.get(), _int8_ffn_out_buf.get(),
                             w.ffn1_act_lut.get(), M, I, H, c[2] * c[6] / (c[10] * Q), _stream));
    act_buf = _int8_ffn_out_buf.get();
  } else {
    prof_begin(2, M, I, H, "EpiI8");
    LSH_CALL(gemm_i8_i8o(_int8_ffn_in_buf.get(), w.w_ffn1.get(), _int8_ffn_out_buf.get(), M, I, H,
                         c[2] * c[6] / (c[10] * Q), _stream));
    tap(taps.ffn1_q, _int8_ffn_out_buf.get(), (size_t)M * I);
    if (_tw._use_gelu) {
      LSH_CALL(bias_gelu_i8I_i8O<__half>(M, _stream, _int8_ffn_out_buf.get(),
                                         _int8_ffn_in_buf.get(), w.b_ffn1.get(), I, c[10] / Q,
                                         Q / c[7]));
    } else {
      LSH_CALL(bias_relu_i8I_i8O<__half>(M, _stream, _int8_ffn_out_buf.get(),
                                         _int8_ffn_in_buf.get(), w.b_ffn1.get(), I, c[10] / Q,
                                         Q / c[7], c[7], true));
    }
  }
  tap(taps.act_q, act_buf, (size_t)M * I);

  prof_begin(3, M, H, I, "EpiI32");
  // K split over workgroups when the tile count would leave compute units idle; the planes
  // are summed (exactly) by the layer-norm kernel that consumes them
  const bool tap_acc = taps.ffn2_acc && taps.tap_layer == _layer_id;
  int nparts = 1;
  LSH_CALL(gemm_i8_i32o_splitk(act_buf, w.w_ffn2.get(), _int32_ffn_out_buf.get(), M, H, I,
                               tap_acc ? 1 : std::min(4, gemm_i8_preferred_ksplit(M, H, I)),
                               &nparts, _stream));
  const long part_stride = (long)M * H;
  if (tap_acc)
    CHECK_GPU_ERROR(hipMemcpyAsync(taps.ffn2_acc, _int32_ffn_out_buf.get(),
                                   (size_t)M * H * sizeof(int32_t), hipMemcpyDeviceToDevice,
                                   _stream));

  if (taps.res_ffn && taps.tap_layer == _layer_id)
    CHECK_GPU_ERROR(hipMemcpyAsync(taps.res_ffn, _p_d_output, (size_t)M * H * sizeof(__half),
                                   hipMemcpyDeviceToDevice, _stream));
  if (last) {
    LSH_CALL(residual_bias_ln_i32I<__half>(_int32_ffn_out_buf.get(), _final_ln_scale.get(),
                                           _final_ln_bias.get(), _p_d_output, _p_d_output, M, H,
                                           dequant_scale, _stream, colsum, nparts, part_stride));
  } else {
    const Layer& nx = _layers[_layer_id + 1];
    const float clip_next = _enc_clip_max[(_layer_id + 1) * _tw._clip_stride + 4];
    LSH_CALL((residual_bias_ln_i8O<__half, int32_t>(
        _int32_ffn_out_buf.get(), nx.ln1_scale.get(), nx.ln1_bias.get(), nx.b_out.get(),
        _int8_ffn_in_buf.get(), _p_d_output, M, H, dequant_scale, Q / clip_next, _stream,
        _tw._is_post_ln, colsum, nparts, part_stride)));
  }
}

}  // namespace hip
}  // namespace lightseq
