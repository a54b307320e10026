// Host orchestration of the int8 BERT encoder stack on one MI355X: device buffers,
// per-layer launch sequence and scale bookkeeping.
//
// Same role and call order as lightseq/inference/model/quant_bert_encoder.{h,cc.cu}
// (init_buffer :52-179, check :185-208, run_one_infer :214-265, self_attention
// :271-399, ffn_add_norm :402-520), fp16 storage.  What differs is how the work is
// mapped to the GPU: hand-written MFMA GEMMs instead of cuBLASLt, one fused attention
// kernel instead of two batched GEMMs + softmax + arrange, and no COL32 layouts.
#pragma once

#include <string>
#include <vector>

#include "model_util.h"
#include "quant_bert_weight.h"

namespace lightseq {
namespace hip {

class QuantBertEncoder {
 public:
  QuantBertEncoder(int max_batch_size, const int* p_d_token_id, int* p_d_padding_mask,
                   __half* p_d_output, const QuantBertWeight& tw, hipStream_t stream);
  ~QuantBertEncoder();
  void init_buffer();
  std::string check();
  void run_one_infer(int batch_size, int batch_seq_len);
  // After the stream has been synchronised: true when the run has to be repeated (a kernel that
  // waits for workgroups of its own launch gave up; the encoder has switched that route off).
  bool finish_infer();

  // Debug taps (all optional, device pointers owned by the caller): copies of the
  // intermediates of layer `tap_layer`, for parity bisection.
  struct Taps {
    int tap_layer = -1;
    int8_t *ln1_q = nullptr, *qkv_q = nullptr, *ctx_q = nullptr, *out_q = nullptr,
           *ln2_q = nullptr, *ffn1_q = nullptr, *act_q = nullptr;
    int32_t* ffn2_acc = nullptr;
    // fp16 residual stream as read by the LayerNorm kernel after the attention
    // out-projection / after FFN2
    __half *res_attn = nullptr, *res_ffn = nullptr;
  } taps;

  // Per-GEMM-site timing with HIP events on the model's stream (off by default).
  // collect_profile() must be called after the stream has been synchronised.
  struct SiteProfile {
    std::string site, kernel, route;
    int m = 0, n = 0, k = 0;
    long launches = 0;
    double total_ms = 0.0;
  };
  void set_profiling(bool on);
  void set_fusion(bool on) { _fuse = on; }
  void collect_profile();
  void reset_profile();
  const std::vector<SiteProfile>& profile() const { return _profile; }

  const int* _p_d_token_id;
  int* _p_d_padding_mask;
  __half* _p_d_output;

 private:
  void self_attention();
  void ffn_add_norm();
  void tap(int8_t* dst, const int8_t* src, size_t n);
  // event bracket around one GEMM launch of `site` (0 qkv, 1 out, 2 ffn1, 3 ffn2)
  void prof_begin(int site, int m, int n, int k, const char* epilogue);
  bool _profiling = false;
  bool _fuse = true;  // use the fused GEMM epilogues (QKV arrange, FFN1 bias+activation)
  std::vector<SiteProfile> _profile;
  struct Pending { int site; hipEvent_t e0, e1; };
  std::vector<Pending> _pending;
  std::vector<hipEvent_t> _event_pool;
  // the feed-forward half of a layer as one launch (xcd_ffn_kernels.hip)
  DeviceBuffer<unsigned> _seg_sync;
  unsigned _seg_launches = 0;
  unsigned* _h_seg_error = nullptr;  // pinned copy of the error word
  bool _seg_active = false;          // this run holds the process-wide claim
  bool _seg_off = false;             // switched off after a launch that gave up

  const int _max_batch_size;
  const QuantBertWeight& _tw;
  hipStream_t _stream;
  const float _quant_range = 127.f;
  const float _src_emb_clip_max;
  const std::vector<float> _enc_clip_max;

  int _batch_size = 0, _batch_seq_len = 0, _batch_token_num = 0, _layer_id = 0;
  long _max_batch_dim;

  // activations
  DeviceBuffer<__half> _qkv_buf;  // q | k | v, each max_batch_dim
  DeviceBuffer<int8_t> _int8_ffn_in_buf, _int8_ffn_out_buf;
  DeviceBuffer<int32_t> _int32_ffn_out_buf;
  DeviceBuffer<int> _qa_plan;      // plan of the fused QKV + attention launches of a call
  const int* _qa_plan_cur = nullptr;  // ... when this call has one
  // weights
  DeviceBuffer<int8_t> _int8_emb;                       // [vocab, H]
  DeviceBuffer<__half> _pos_emb, _final_ln_scale, _final_ln_bias;
  struct Layer {
    DeviceBuffer<int8_t> w_qkv, w_out, w_ffn1, w_ffn2;  // [N, K] int8
    DeviceBuffer<int8_t> w_out_tiled;  // w_out in 16 x 64 MFMA tiles (fused out-projection + LN)
    DeviceBuffer<int8_t> ffn1_act_lut;  // [inner, 256]: bias + activation + requant per code
    DeviceBuffer<__half> ln1_scale, ln1_bias, b_qkv, b_out, ln2_scale, ln2_bias, b_ffn1, b_ffn2,
        ffn2_colsum;
  };
  std::vector<Layer> _layers;
};

}  // namespace hip
}  // namespace lightseq
