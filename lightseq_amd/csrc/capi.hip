// extern "C" surface of the library: argument validation, status/error plumbing and
// dispatch on the storage type.  No kernel code lives here.
#include <string>

#include "ls_device.h"
#include "ls_launch.h"

namespace lsh {

static thread_local std::string g_last_error;

int lsh_fail(int code, const char* msg) {
  g_last_error = msg ? msg : "";
  return code;
}

int lsh_check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return LSH_OK;
  g_last_error = std::string(what ? what : "hip") + ": " + hipGetErrorName(e) + " " +
                 hipGetErrorString(e);
  return LSH_ERR_HIP;
}

int lsh_check_launch(const char* what) { return lsh_check_hip(hipGetLastError(), what); }

static int no_col32(int flag_a, int flag_b, const char* who) {
  if (flag_a || flag_b) {
    g_last_error = std::string(who) + ": COL32 layouts are cuBLASLt-specific and not provided";
    return LSH_ERR_UNSUPPORTED;
  }
  return LSH_OK;
}

template <typename T>
static int quantize_weight_impl(const void* host_w, int8_t* dev_q, int rows, int cols,
                                float quant_scale, hipStream_t s, int layout) {
  if (!host_w || !dev_q || rows <= 0 || cols <= 0)
    return lsh_fail(LSH_ERR_INVALID, "quantize_weight: bad arguments");
  if (layout != 0 && layout != 1)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "unsupported layout");
  T* tmp = nullptr;
  const size_t bytes = (size_t)rows * cols * sizeof(T);
  int rc = lsh_check_hip(hipMalloc(&tmp, bytes), "hipMalloc(quantize_weight)");
  if (rc) return rc;
  rc = lsh_check_hip(hipMemcpyAsync(tmp, host_w, bytes, hipMemcpyHostToDevice, s),
                     "hipMemcpyAsync(quantize_weight)");
  if (!rc) rc = quantize_transpose<T>(tmp, dev_q, rows, cols, quant_scale, layout == 1, s);
  hipError_t e = hipStreamSynchronize(s);
  if (!rc) rc = lsh_check_hip(e, "hipStreamSynchronize(quantize_weight)");
  (void)hipFree(tmp);
  return rc;
}

}  // namespace lsh

using namespace lsh;

#define HS(s) reinterpret_cast<hipStream_t>(s)
#define H(p) reinterpret_cast<const __half*>(p)
#define HM(p) reinterpret_cast<__half*>(p)
#define F(p) reinterpret_cast<const float*>(p)
#define FM(p) reinterpret_cast<float*>(p)

extern "C" {

const char* lsh_last_error(void) { return g_last_error.c_str(); }
const char* lsh_version(void) { return "lightseq_hip 0.1 (gfx950)"; }

// ---- quantise / dequantise ------------------------------------------------------
int lsh_launch_quantize_tensor_f16(const void* input, int8_t* output, int batch_tokens,
                                   int hidden_size, float quant_scale, lsh_stream_t stream,
                                   int out_col32) {
  if (int rc = no_col32(out_col32, 0, "launch_quantize_tensor")) return rc;
  if (batch_tokens < 0 || hidden_size < 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_quantize_tensor: negative shape");
  return quantize_tensor<__half>(H(input), output, (long)batch_tokens * hidden_size, quant_scale,
                                 HS(stream));
}
int lsh_launch_quantize_tensor_f32(const void* input, int8_t* output, int batch_tokens,
                                   int hidden_size, float quant_scale, lsh_stream_t stream,
                                   int out_col32) {
  if (int rc = no_col32(out_col32, 0, "launch_quantize_tensor")) return rc;
  if (batch_tokens < 0 || hidden_size < 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_quantize_tensor: negative shape");
  return quantize_tensor<float>(F(input), output, (long)batch_tokens * hidden_size, quant_scale,
                                HS(stream));
}
int lsh_launch_dequantize_tensor_f16(const int32_t* input, void* output, int batch_tokens,
                                     int hidden_size, float dequant_scale, lsh_stream_t stream,
                                     int in_col32) {
  if (int rc = no_col32(in_col32, 0, "launch_dequantize_tensor")) return rc;
  if (batch_tokens < 0 || hidden_size < 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_dequantize_tensor: negative shape");
  return dequantize_tensor<__half>(input, HM(output), (long)batch_tokens * hidden_size,
                                   dequant_scale, HS(stream));
}
int lsh_launch_dequantize_tensor_f32(const int32_t* input, void* output, int batch_tokens,
                                     int hidden_size, float dequant_scale, lsh_stream_t stream,
                                     int in_col32) {
  if (int rc = no_col32(in_col32, 0, "launch_dequantize_tensor")) return rc;
  if (batch_tokens < 0 || hidden_size < 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_dequantize_tensor: negative shape");
  return dequantize_tensor<float>(input, FM(output), (long)batch_tokens * hidden_size,
                                  dequant_scale, HS(stream));
}

int lsh_dec_emb_norm_layer_i8O_f16(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                                   void* residual, int8_t* out_q, const void* scale,
                                   const void* bias, const void* residual_bias, int rows,
                                   int hidden, int vocab_size, int step, int max_step,
                                   float dequant_scale, int scaled, float quant_scale,
                                   int is_post_ln, lsh_stream_t stream) {
  return dec_emb_norm_layer_i8O<__half>(token_emb, H(pos_emb), tokens, HM(residual), out_q, H(scale),
                                        H(bias), H(residual_bias), rows, hidden, vocab_size, step,
                                        max_step, dequant_scale, scaled != 0, quant_scale,
                                        is_post_ln != 0, HS(stream));
}
int lsh_gpt_emb_step_norm_layer_i8O_f16(const int8_t* token_emb, const void* pos_emb,
                                        const int* token_id, void* residual, int8_t* out_q,
                                        const void* scale, const void* bias,
                                        const void* residual_bias, int* real_seq_len,
                                        int* zero_flag, int batch_size, int hidden, int vocab_size,
                                        int padding_id, int pos, int max_step, float dequant_scale,
                                        float quant_scale, int is_post_ln, lsh_stream_t stream) {
  return gpt_emb_step_norm_layer_i8O<__half>(
      token_emb, H(pos_emb), token_id, HM(residual), out_q, H(scale), H(bias), H(residual_bias),
      real_seq_len, zero_flag, batch_size, hidden, vocab_size, padding_id, pos, max_step,
      dequant_scale, quant_scale, is_post_ln != 0, HS(stream));
}
// ---- LayerNorm family --------------------------------------------------------------
int lsh_layer_norm_row_kernel(int on) { return ln_set_few_rows(on != 0) ? 1 : 0; }
int lsh_gemm_i8_tile_kernel(int on) { return gemm_i8_enable_tile_kernel(on != 0) ? 1 : 0; }
int lsh_gemm_i8_decode_kernel_16x16(int on) {
  return gemm_i8_enable_skinny16_kernel(on != 0) ? 1 : 0;
}
int lsh_bias_act_lut_kernel(int on) { return bias_act_enable_lut_kernel(on != 0) ? 1 : 0; }
int lsh_tile_weight_16x64(const int8_t* w, int8_t* tiled, int n, int k, lsh_stream_t stream) {
  return tile_weight_16x64(w, tiled, n, k, HS(stream));
}
int lsh_gemm_i8_residual_ln_i8O_f16(const int8_t* A, const int8_t* w_tiled, float alpha,
                                    const void* scale, const void* bias, const void* residual_bias,
                                    int8_t* output, void* residual, int batch_tokens,
                                    int hidden_size, int k, float dequant_scale, float quant_scale,
                                    lsh_stream_t stream, int is_post_ln) {
  return gemm_i8_residual_ln_i8O<__half>(A, w_tiled, alpha, H(scale), H(bias), H(residual_bias),
                                         output, HM(residual), batch_tokens, hidden_size, k,
                                         dequant_scale, quant_scale, HS(stream), is_post_ln != 0);
}
int lsh_ffn_segment_in_models(int on) { return ffn_segment_enable(on != 0) ? 1 : 0; }
int lsh_ffn_segment_stamps(uint64_t* dev) {
  ffn_segment_stamps(reinterpret_cast<unsigned long long*>(dev));
  return LSH_OK;
}
size_t lsh_ffn_segment_sync_words(void) { return ffn_segment_sync_words(); }
int lsh_ffn_segment_supported(int m, int hidden, int inner) {
  return ffn_segment_supported(m, hidden, inner) ? 1 : 0;
}
int lsh_ffn_segment_i8_f16(const int8_t* x, const int8_t* w1, const int8_t* lut1, float alpha1,
                           int8_t* act, const int8_t* w2, int32_t* acc, void* residual, void* out_t,
                           int8_t* out_q, const void* scale, const void* bias,
                           const void* residual_bias, const void* colsum, int m, int hidden,
                           int inner, float dequant_scale, float quant_scale, int is_post_ln,
                           int final_ln, uint32_t* sync, uint32_t* launches, int spin_limit,
                           lsh_stream_t stream) {
  return ffn_segment_i8(x, w1, lut1, alpha1, act, w2, acc, HM(residual), HM(out_t), out_q, H(scale),
                        H(bias), H(residual_bias), H(colsum), m, hidden, inner, dequant_scale,
                        quant_scale, is_post_ln != 0, final_ln != 0, sync, launches, spin_limit,
                        HS(stream));
}
int lsh_mfma_i8_peak_probe(int* out, int workgroups, int iters, double* ops, lsh_stream_t stream) {
  return mfma_i8_peak_probe(out, workgroups, iters, ops, HS(stream));
}
int lsh_ker_norm_layer_resual_i8O_f16(int token_num, int hidden_size, lsh_stream_t stream,
                                      void* input, int8_t* output, const void* scale,
                                      const void* bias, const void* residual_bias,
                                      int /*max_thread_per_block*/, float quant_scale,
                                      int is_post_ln, int out_col32) {
  if (int rc = no_col32(out_col32, 0, "ker_norm_layer_resual_i8O")) return rc;
  return norm_layer_resual_i8O<__half>(token_num, hidden_size, HS(stream), HM(input), output,
                                       H(scale), H(bias), H(residual_bias), quant_scale,
                                       is_post_ln != 0);
}
int lsh_ker_norm_layer_resual_i8O_f32(int token_num, int hidden_size, lsh_stream_t stream,
                                      void* input, int8_t* output, const void* scale,
                                      const void* bias, const void* residual_bias,
                                      int /*max_thread_per_block*/, float quant_scale,
                                      int is_post_ln, int out_col32) {
  if (int rc = no_col32(out_col32, 0, "ker_norm_layer_resual_i8O")) return rc;
  return norm_layer_resual_i8O<float>(token_num, hidden_size, HS(stream), FM(input), output,
                                      F(scale), F(bias), F(residual_bias), quant_scale,
                                      is_post_ln != 0);
}

#define LSH_RES_LN(NAME, ACC, SUFFIX, T, CT, MT)                                                \
  int NAME##SUFFIX(const ACC* input, const void* scale, const void* bias,                       \
                   const void* residual_bias, int8_t* output, void* residual, int batch_tokens, \
                   int hidden_size, float dequant_scale, float quant_scale,                     \
                   int /*max_thread_per_block*/, lsh_stream_t stream, int is_post_ln,           \
                   int in_col32, int out_col32, const void* colsum) {                           \
    if (int rc = no_col32(in_col32, out_col32, #NAME)) return rc;                               \
    return residual_bias_ln_i8O<T, ACC>(input, CT(scale), CT(bias), CT(residual_bias), output,  \
                                        MT(residual), batch_tokens, hidden_size, dequant_scale, \
                                        quant_scale, HS(stream), is_post_ln != 0, CT(colsum));  \
  }
LSH_RES_LN(lsh_ker_residual_bias_ln_i32I_i8O, int32_t, _f16, __half, H, HM)
LSH_RES_LN(lsh_ker_residual_bias_ln_i32I_i8O, int32_t, _f32, float, F, FM)
LSH_RES_LN(lsh_ker_residual_bias_ln_i8I_i8O, int8_t, _f16, __half, H, HM)
LSH_RES_LN(lsh_ker_residual_bias_ln_i8I_i8O, int8_t, _f32, float, F, FM)
#undef LSH_RES_LN

int lsh_ker_residual_bias_ln_i32I_f16(const int32_t* input, const void* scale, const void* bias,
                                      const void* residual, void* output, int batch_tokens,
                                      int hidden_size, float dequant_scale,
                                      int /*max_thread_per_block*/, lsh_stream_t stream,
                                      int in_col32, const void* colsum) {
  if (int rc = no_col32(in_col32, 0, "ker_residual_bias_ln_i32I")) return rc;
  return residual_bias_ln_i32I<__half>(input, H(scale), H(bias), H(residual), HM(output),
                                       batch_tokens, hidden_size, dequant_scale, HS(stream),
                                       H(colsum));
}
int lsh_ker_residual_bias_ln_i32I_f32(const int32_t* input, const void* scale, const void* bias,
                                      const void* residual, void* output, int batch_tokens,
                                      int hidden_size, float dequant_scale,
                                      int /*max_thread_per_block*/, lsh_stream_t stream,
                                      int in_col32, const void* colsum) {
  if (int rc = no_col32(in_col32, 0, "ker_residual_bias_ln_i32I")) return rc;
  return residual_bias_ln_i32I<float>(input, F(scale), F(bias), F(residual), FM(output),
                                      batch_tokens, hidden_size, dequant_scale, HS(stream),
                                      F(colsum));
}

// ---- bias + activation + requant ------------------------------------------------------
int lsh_ker_bias_gelu_i8I_i8O_f16(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, int in_col32,
                                  int out_col32) {
  if (int rc = no_col32(in_col32, out_col32, "ker_bias_gelu_i8I_i8O")) return rc;
  return bias_gelu_i8I_i8O<__half>(batch_token_num, HS(stream), input, output, H(bias),
                                   feature_dim, dequant_scale, quant_scale);
}
int lsh_ker_bias_gelu_i8I_i8O_f32(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, int in_col32,
                                  int out_col32) {
  if (int rc = no_col32(in_col32, out_col32, "ker_bias_gelu_i8I_i8O")) return rc;
  return bias_gelu_i8I_i8O<float>(batch_token_num, HS(stream), input, output, F(bias),
                                  feature_dim, dequant_scale, quant_scale);
}
int lsh_ker_bias_relu_i8I_i8O_f16(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, float clip_max,
                                  int in_col32, int out_col32, int narrow_clip) {
  if (int rc = no_col32(in_col32, out_col32, "ker_bias_relu_i8I_i8O")) return rc;
  return bias_relu_i8I_i8O<__half>(batch_token_num, HS(stream), input, output, H(bias),
                                   feature_dim, dequant_scale, quant_scale, clip_max,
                                   narrow_clip != 0);
}
int lsh_ker_bias_relu_i8I_i8O_f32(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, float clip_max,
                                  int in_col32, int out_col32, int narrow_clip) {
  if (int rc = no_col32(in_col32, out_col32, "ker_bias_relu_i8I_i8O")) return rc;
  return bias_relu_i8I_i8O<float>(batch_token_num, HS(stream), input, output, F(bias),
                                  feature_dim, dequant_scale, quant_scale, clip_max,
                                  narrow_clip != 0);
}

// ---- head split / merge -------------------------------------------------------------------
int lsh_ker_arrange_encself_qkv_i8I_f16(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                        const int8_t* ori_qkv, const void* qkv_bias, void* new_qkv,
                                        int max_batch_dim, int batch_seq_len, int dim_per_head,
                                        int head_num, int /*max_thread_per_block*/,
                                        float dequant_scale, int in_col32) {
  if (int rc = no_col32(in_col32, 0, "ker_arrange_encself_qkv_i8I")) return rc;
  return arrange_encself_qkv_i8I<__half>(batch_token_num, hidden_size, HS(stream), ori_qkv,
                                         H(qkv_bias), HM(new_qkv), max_batch_dim, batch_seq_len,
                                         dim_per_head, head_num, dequant_scale);
}
int lsh_ker_arrange_encself_qkv_i8I_f32(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                        const int8_t* ori_qkv, const void* qkv_bias, void* new_qkv,
                                        int max_batch_dim, int batch_seq_len, int dim_per_head,
                                        int head_num, int /*max_thread_per_block*/,
                                        float dequant_scale, int in_col32) {
  if (int rc = no_col32(in_col32, 0, "ker_arrange_encself_qkv_i8I")) return rc;
  return arrange_encself_qkv_i8I<float>(batch_token_num, hidden_size, HS(stream), ori_qkv,
                                        F(qkv_bias), FM(new_qkv), max_batch_dim, batch_seq_len,
                                        dim_per_head, head_num, dequant_scale);
}
int lsh_ker_arrange_encself_qkv_i8I_i8O_f16(int batch_token_num, int hidden_size,
                                            lsh_stream_t stream, const int8_t* ori_qkv,
                                            const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                            int8_t* new_v, void* d_v, int batch_seq_len,
                                            int dim_per_head, int head_num,
                                            int /*max_thread_per_block*/, float dequant_scale,
                                            float quant_scale, int in_col32) {
  if (int rc = no_col32(in_col32, 0, "ker_arrange_encself_qkv_i8I_i8O")) return rc;
  return arrange_encself_qkv_i8I_i8O<__half>(batch_token_num, hidden_size, HS(stream), ori_qkv,
                                             H(qkv_bias), new_q, new_k, new_v, HM(d_v),
                                             batch_seq_len, dim_per_head, head_num, dequant_scale,
                                             quant_scale);
}
int lsh_ker_arrange_encself_qkv_i8I_i8O_f32(int batch_token_num, int hidden_size,
                                            lsh_stream_t stream, const int8_t* ori_qkv,
                                            const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                            int8_t* new_v, void* d_v, int batch_seq_len,
                                            int dim_per_head, int head_num,
                                            int /*max_thread_per_block*/, float dequant_scale,
                                            float quant_scale, int in_col32) {
  if (int rc = no_col32(in_col32, 0, "ker_arrange_encself_qkv_i8I_i8O")) return rc;
  return arrange_encself_qkv_i8I_i8O<float>(batch_token_num, hidden_size, HS(stream), ori_qkv,
                                            F(qkv_bias), new_q, new_k, new_v, FM(d_v),
                                            batch_seq_len, dim_per_head, head_num, dequant_scale,
                                            quant_scale);
}
int lsh_ker_arrange_atten_output_i8O_f16(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                         const void* ori_q, int8_t* new_q, int beam_size,
                                         int dim_per_head, int head_num,
                                         int /*max_thread_per_block*/, float quant_scale,
                                         int out_col32) {
  if (int rc = no_col32(out_col32, 0, "ker_arrange_atten_output_i8O")) return rc;
  return arrange_atten_output_i8O<__half>(batch_token_num, hidden_size, HS(stream), H(ori_q),
                                          new_q, beam_size, dim_per_head, head_num, quant_scale);
}
int lsh_ker_arrange_atten_output_i8O_f32(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                         const void* ori_q, int8_t* new_q, int beam_size,
                                         int dim_per_head, int head_num,
                                         int /*max_thread_per_block*/, float quant_scale,
                                         int out_col32) {
  if (int rc = no_col32(out_col32, 0, "ker_arrange_atten_output_i8O")) return rc;
  return arrange_atten_output_i8O<float>(batch_token_num, hidden_size, HS(stream), F(ori_q), new_q,
                                         beam_size, dim_per_head, head_num, quant_scale);
}

// ---- encoder attention core ------------------------------------------------------------------
int lsh_ker_correlation_softmax_encself_f16(int batch_size, int batch_seq_len, int head_num,
                                            lsh_stream_t stream, void* correlation,
                                            const int* src_padding_mask) {
  return correlation_softmax_encself<__half>(batch_size, batch_seq_len, head_num, HS(stream),
                                             HM(correlation), src_padding_mask);
}
int lsh_ker_correlation_softmax_encself_f32(int batch_size, int batch_seq_len, int head_num,
                                            lsh_stream_t stream, void* correlation,
                                            const int* src_padding_mask) {
  return correlation_softmax_encself<float>(batch_size, batch_seq_len, head_num, HS(stream),
                                            FM(correlation), src_padding_mask);
}
int lsh_encself_attention_f16(const void* q, const void* k, const void* v,
                              const int* src_padding_mask, void* ctx, int8_t* ctx_q,
                              float quant_scale, int batch_size, int batch_seq_len, int head_num,
                              int dim_per_head, lsh_stream_t stream) {
  return encself_attention_f16(H(q), H(k), H(v), src_padding_mask, HM(ctx), ctx_q, quant_scale,
                               batch_size, batch_seq_len, head_num, dim_per_head, HS(stream));
}
int lsh_encself_attention_i8qkv_f16(const int8_t* qkv, const void* qkv_bias, float dequant_scale,
                                    const int* src_padding_mask, void* ctx, int8_t* ctx_q,
                                    float quant_scale, int batch_size, int batch_seq_len,
                                    int head_num, int dim_per_head, lsh_stream_t stream) {
  return encself_attention_i8qkv(qkv, H(qkv_bias), dequant_scale, src_padding_mask, HM(ctx), ctx_q,
                                 quant_scale, batch_size, batch_seq_len, head_num, dim_per_head,
                                 HS(stream));
}

int lsh_qkv_attention_i8_f16(const int8_t* x, const int8_t* qkv_weight, const void* qkv_bias,
                             const int* src_padding_mask, int8_t* ctx_q, float requant_alpha,
                             float dequant_scale, float quant_scale, int batch_size,
                             int batch_seq_len, int head_num, int dim_per_head,
                             lsh_stream_t stream) {
  return qkv_attention_i8(x, qkv_weight, H(qkv_bias), src_padding_mask, ctx_q, requant_alpha,
                          dequant_scale, quant_scale, batch_size, batch_seq_len, head_num,
                          dim_per_head, HS(stream));
}

int lsh_qkv_attention_plan_in_models(int on) { return qkv_attention_plan_enable(on != 0) ? 1 : 0; }
int lsh_qkv_attention_plan(const int* src_padding_mask, int* plan, int batch_size,
                           int batch_seq_len, int head_num, lsh_stream_t stream) {
  return qkv_attention_plan(src_padding_mask, plan, batch_size, batch_seq_len, head_num, HS(stream));
}
int lsh_qkv_attention_planned_i8_f16(const int8_t* x, const int8_t* qkv_weight, const void* qkv_bias,
                                     const int* src_padding_mask, const int* plan, int8_t* ctx_q,
                                     float requant_alpha, float dequant_scale, float quant_scale,
                                     int batch_size, int batch_seq_len, int head_num,
                                     int dim_per_head, lsh_stream_t stream) {
  if (!plan) return lsh_fail(LSH_ERR_INVALID, "qkv_attention_planned_i8: null plan");
  return qkv_attention_i8(x, qkv_weight, H(qkv_bias), src_padding_mask, ctx_q, requant_alpha,
                          dequant_scale, quant_scale, batch_size, batch_seq_len, head_num,
                          dim_per_head, HS(stream), plan);
}

// ---- embedding ----------------------------------------------------------------------------------
int lsh_launch_enc_emb_i8I_f16(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               void* output, int* pad_mask, int pad_id, int batch_size,
                               int seq_len, int hidden_dim, lsh_stream_t stream,
                               const void* /*lang_emb*/, const int* /*lang_id*/, int multilg_type,
                               float dequant_scale, int scaled) {
  if (multilg_type != 0) return lsh_fail(LSH_ERR_INVALID, "multilingle not supported");
  return enc_emb_i8I<__half>(token_emb, H(pos_emb), tokens, HM(output), pad_mask, pad_id,
                             batch_size, seq_len, hidden_dim, HS(stream), dequant_scale,
                             scaled != 0, 0);
}
int lsh_launch_enc_emb_i8I_f32(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               void* output, int* pad_mask, int pad_id, int batch_size,
                               int seq_len, int hidden_dim, lsh_stream_t stream,
                               const void* /*lang_emb*/, const int* /*lang_id*/, int multilg_type,
                               float dequant_scale, int scaled) {
  if (multilg_type != 0) return lsh_fail(LSH_ERR_INVALID, "multilingle not supported");
  return enc_emb_i8I<float>(token_emb, F(pos_emb), tokens, FM(output), pad_mask, pad_id,
                            batch_size, seq_len, hidden_dim, HS(stream), dequant_scale,
                            scaled != 0, 0);
}
int lsh_launch_scaled_colsum_f16(const void* inp, void* out, int rows, int cols, float scale,
                                 lsh_stream_t stream) {
  return scaled_colsum<__half>(H(inp), HM(out), rows, cols, scale, HS(stream));
}
int lsh_launch_scaled_colsum_f32(const void* inp, void* out, int rows, int cols, float scale,
                                 lsh_stream_t stream) {
  return scaled_colsum<float>(F(inp), FM(out), rows, cols, scale, HS(stream));
}

// ---- int8 GEMM --------------------------------------------------------------------------------------
int lsh_gemm_i8_i32o(const int8_t* A, const int8_t* W, int32_t* C, int m, int n, int k,
                     lsh_stream_t stream) {
  return gemm_i8_i32o(A, W, C, m, n, k, HS(stream));
}
int lsh_build_act_lut(int8_t* lut, const void* bias_f16, int n, float dequant_scale,
                      float quant_scale, float clip_max, int act, lsh_stream_t stream) {
  return build_act_lut(lut, H(bias_f16), n, dequant_scale, quant_scale, clip_max, act, HS(stream));
}
int lsh_gemm_i8_decself_qkv_i8o_f16(const int8_t* A, const int8_t* W, const void* qkv_bias,
                                    int8_t* new_q, int8_t* new_k, int8_t* new_v,
                                    int step_token_num, int hidden, int k, int head_num,
                                    int max_step, int step_id, float alpha, float dequant_scale,
                                    float quant_scale, lsh_stream_t stream) {
  return gemm_i8_decself_qkv_i8o(A, W, H(qkv_bias), new_q, new_k, new_v, step_token_num, hidden, k,
                                 head_num, max_step, step_id, alpha, dequant_scale, quant_scale,
                                 HS(stream));
}
int lsh_decself_qkv_attention_in_models(int on) {
  return decself_qkv_attention_enable(on != 0) ? 1 : 0;
}
int lsh_decself_qkv_attention_i8_f16(const int8_t* x, const int8_t* qkv_weight,
                                     const void* qkv_bias, int8_t* new_q, int8_t* k_cache,
                                     int8_t* v_cache, int8_t* ctx, int rows, int hidden,
                                     int head_num, int max_step, int step_id, float alpha,
                                     float dequant_scale, float cache_quant_scale,
                                     float attn_scale, float cache_dequant_scale,
                                     float ctx_quant_scale, lsh_stream_t stream) {
  return decself_qkv_attention_i8(x, qkv_weight, H(qkv_bias), new_q, k_cache, v_cache, ctx, rows,
                                  hidden, head_num, max_step, step_id, alpha, dequant_scale,
                                  cache_quant_scale, attn_scale, cache_dequant_scale,
                                  ctx_quant_scale, HS(stream));
}
int lsh_gemm_i8_encdec_q_f16(const int8_t* A, const int8_t* W, const void* q_bias, void* new_q,
                             int step_token_num, int hidden, int k, int beam_size, int head_num,
                             float alpha, float dequant_scale, lsh_stream_t stream) {
  return gemm_i8_encdec_q_f16(A, W, H(q_bias), HM(new_q), step_token_num, hidden, k, beam_size,
                              head_num, alpha, dequant_scale, HS(stream));
}
int lsh_encdec_q_attention_f16(const int8_t* x, const int8_t* q_weight, const void* q_bias,
                               const void* k, const void* v, const int* pad_mask, int8_t* ctx_q,
                               float quant_scale, int batch_size, int beam_size, int head_num,
                               int batch_seq_len, int hidden, float alpha, float dequant_scale,
                               lsh_stream_t stream) {
  return encdec_q_attention_f16(x, q_weight, H(q_bias), H(k), H(v), pad_mask, ctx_q, quant_scale,
                                batch_size, beam_size, head_num, batch_seq_len, hidden, alpha,
                                dequant_scale, HS(stream));
}
int lsh_gemm_i8_lut_i8o(const int8_t* A, const int8_t* W, int8_t* C, const int8_t* lut, int m,
                        int n, int k, float alpha, lsh_stream_t stream) {
  return gemm_i8_lut_i8o(A, W, C, lut, m, n, k, alpha, HS(stream));
}
int lsh_gemm_i8_i32o_splitk(const int8_t* A, const int8_t* W, int32_t* C, int m, int n, int k,
                            int ksplit, int* used, lsh_stream_t stream) {
  return gemm_i8_i32o_splitk(A, W, C, m, n, k, ksplit, used, HS(stream));
}
int lsh_gemm_i8_preferred_ksplit(int m, int n, int k) { return gemm_i8_preferred_ksplit(m, n, k); }
int lsh_ker_residual_bias_ln_planes_i32I_i8O_f16(const int32_t* input, int nparts,
                                                 int64_t part_stride, const void* scale,
                                                 const void* bias, const void* residual_bias,
                                                 int8_t* output, void* residual, int batch_tokens,
                                                 int hidden_size, float dequant_scale,
                                                 float quant_scale, lsh_stream_t stream,
                                                 int is_post_ln, const void* colsum) {
  return residual_bias_ln_i8O<__half, int32_t>(input, H(scale), H(bias), H(residual_bias), output,
                                               HM(residual), batch_tokens, hidden_size,
                                               dequant_scale, quant_scale, HS(stream),
                                               is_post_ln != 0, H(colsum), nparts,
                                               (long)part_stride);
}
int lsh_gemm_i8_i8o(const int8_t* A, const int8_t* W, int8_t* C, int m, int n, int k, float alpha,
                    lsh_stream_t stream) {
  return gemm_i8_i8o(A, W, C, m, n, k, alpha, HS(stream));
}
int lsh_gemm_i8_bias_gelu_i8o_f16(const int8_t* A, const int8_t* W, int8_t* C, const void* bias,
                                  int m, int n, int k, float alpha, float dequant_scale,
                                  float quant_scale, lsh_stream_t stream) {
  return gemm_i8_bias_act_i8o(A, W, C, H(bias), m, n, k, alpha, dequant_scale, quant_scale, 0.f,
                              kActGelu, HS(stream));
}
int lsh_gemm_i8_bias_relu_i8o_f16(const int8_t* A, const int8_t* W, int8_t* C, const void* bias,
                                  int m, int n, int k, float alpha, float dequant_scale,
                                  float quant_scale, float clip_max, int narrow_clip,
                                  lsh_stream_t stream) {
  return gemm_i8_bias_act_i8o(A, W, C, H(bias), m, n, k, alpha, dequant_scale, quant_scale,
                              clip_max, narrow_clip ? kActReluNarrow : kActRelu, HS(stream));
}
int lsh_gemm_i8_qkv_arrange_f16(const int8_t* A, const int8_t* W, void* new_qkv,
                                const void* qkv_bias, int max_batch_dim, int batch_token_num,
                                int hidden_size, int k, int batch_seq_len, int head_num,
                                float alpha, float dequant_scale, lsh_stream_t stream) {
  return gemm_i8_qkv_arrange_f16(A, W, HM(new_qkv), H(qkv_bias), max_batch_dim, batch_token_num,
                                 hidden_size, k, batch_seq_len, head_num, alpha, dequant_scale,
                                 HS(stream));
}
int lsh_quantize_weight_f16(const void* origin_weight, int8_t* quantized_weight, int rows,
                            int cols, float quant_scale, lsh_stream_t stream, int layout) {
  return quantize_weight_impl<__half>(origin_weight, quantized_weight, rows, cols, quant_scale,
                                      HS(stream), layout);
}
int lsh_quantize_weight_f32(const void* origin_weight, int8_t* quantized_weight, int rows,
                            int cols, float quant_scale, lsh_stream_t stream, int layout) {
  return quantize_weight_impl<float>(origin_weight, quantized_weight, rows, cols, quant_scale,
                                     HS(stream), layout);
}

// ---- decoder step ------------------------------------------------------------------
#define LSH_DEC_EMB(NAME, TY, CAST_C, CAST_M, VM)                                              \
  int NAME(const int8_t* token_emb, const void* pos_emb, const int* tokens,                    \
           const void* lang_emb, const int* lang_id, void* output, int batch_size,             \
           int beam_size, int hidden_dim, int vocab_size, int step, int max_step,              \
           int multilg_type, lsh_stream_t stream, float dequant_scale, int scaled) {           \
    (void)lang_emb;                                                                            \
    (void)lang_id;                                                                             \
    if (multilg_type != 0) return lsh_fail(LSH_ERR_UNSUPPORTED, "multilingle not supported");  \
    return dec_emb_i8I<TY>(token_emb, CAST_C(pos_emb), tokens, CAST_M(output), batch_size,     \
                           beam_size, hidden_dim, vocab_size, step, max_step, HS(stream),      \
                           dequant_scale, scaled != 0, VM);                                    \
  }
LSH_DEC_EMB(lsh_launch_dec_emb_i8I_f16, __half, H, HM, false)
LSH_DEC_EMB(lsh_launch_dec_emb_i8I_f32, float, F, FM, false)
LSH_DEC_EMB(lsh_launch_dec_emb_i8I_vocab_major_f16, __half, H, HM, true)
LSH_DEC_EMB(lsh_launch_dec_emb_i8I_vocab_major_f32, float, F, FM, true)
#undef LSH_DEC_EMB

#define LSH_DECSELF_QKV(NAME, TY, CAST_C)                                                      \
  int NAME(int step_token_num, int hidden_size, lsh_stream_t stream, const int8_t* ori_qkv,    \
           const void* qkv_bias, int8_t* new_q, int8_t* new_k, int8_t* new_v, int head_num,    \
           int dim_per_head, int max_step, int step_id, int max_thread_per_block,              \
           float dequant_scale, float quant_scale, int in_col32) {                             \
    (void)max_thread_per_block;                                                                \
    if (int rc = no_col32(in_col32, 0, "ker_arrange_decself_qkv_i8I_i8O")) return rc;          \
    return arrange_decself_qkv_i8I_i8O<TY>(step_token_num, hidden_size, HS(stream), ori_qkv,   \
                                           CAST_C(qkv_bias), new_q, new_k, new_v, head_num,    \
                                           dim_per_head, max_step, step_id, dequant_scale,     \
                                           quant_scale);                                       \
  }
LSH_DECSELF_QKV(lsh_ker_arrange_decself_qkv_i8I_i8O_f16, __half, H)
LSH_DECSELF_QKV(lsh_ker_arrange_decself_qkv_i8I_i8O_f32, float, F)
#undef LSH_DECSELF_QKV

int lsh_decself_scores_i8_i32o(const int8_t* k_cache, const int8_t* q, int32_t* scores,
                               int batch_head_num, int step_num, int max_step, int dim_per_head,
                               lsh_stream_t stream) {
  return decself_scores_i8(q, k_cache, scores, batch_head_num, step_num, max_step, dim_per_head,
                           HS(stream));
}
int lsh_ker_fuse_softmax_new_value_i32I_i8O(const int32_t* correlation, const int8_t* v,
                                            int8_t* new_v, int batch_head_num, int step_num,
                                            int max_step, int head_num, int dim_per_head,
                                            float attn_scale, float dequant_scale,
                                            float quant_scale, int out_col32,
                                            lsh_stream_t stream) {
  if (int rc = no_col32(out_col32, 0, "ker_fuse_softmax_new_value_i32I_i8O")) return rc;
  return fuse_softmax_new_value_i32I_i8O(correlation, v, new_v, batch_head_num, step_num,
                                         max_step, head_num, dim_per_head, attn_scale,
                                         dequant_scale, quant_scale, HS(stream));
}
int lsh_decself_attention_i8(const int8_t* q, const int8_t* k_cache, const int8_t* v_cache,
                             int8_t* new_v, int batch_head_num, int step_num, int max_step,
                             int head_num, int dim_per_head, float attn_scale,
                             float dequant_scale, float quant_scale, lsh_stream_t stream) {
  return decself_attention_i8(q, k_cache, v_cache, new_v, batch_head_num, step_num, max_step,
                              head_num, dim_per_head, attn_scale, dequant_scale, quant_scale,
                              HS(stream));
}

#define LSH_ENCDEC_Q(NAME, TY, CAST_C, CAST_M)                                                 \
  int NAME(int step_token_num, int hidden_size, lsh_stream_t stream, const int8_t* ori_q,      \
           const void* q_bias, void* new_q, int beam_size, int dim_per_head, int head_num,     \
           int max_thread_per_block, float dequant_scale, int in_col32) {                      \
    (void)max_thread_per_block;                                                                \
    if (int rc = no_col32(in_col32, 0, "ker_arrange_encdec_q_i8I")) return rc;                 \
    return arrange_encdec_q_i8I<TY>(step_token_num, hidden_size, HS(stream), ori_q,            \
                                    CAST_C(q_bias), CAST_M(new_q), beam_size, dim_per_head,    \
                                    head_num, dequant_scale);                                  \
  }
LSH_ENCDEC_Q(lsh_ker_arrange_encdec_q_i8I_f16, __half, H, HM)
LSH_ENCDEC_Q(lsh_ker_arrange_encdec_q_i8I_f32, float, F, FM)
#undef LSH_ENCDEC_Q

#define LSH_ENCDEC_KV(NAME, TY, CAST_C, CAST_M)                                                \
  int NAME(int batch_token_num, int dec_layer_num, int hidden_size, lsh_stream_t stream,       \
           const void* ori_kv, const void* kv_bias, void* new_k, void* new_v,                  \
           int64_t offset_per_layer, int batch_seq_len, int dim_per_head, int head_num,        \
           int max_thread_per_block) {                                                         \
    (void)max_thread_per_block;                                                                \
    return arrange_encdec_kv<TY>(batch_token_num, dec_layer_num, hidden_size, HS(stream),      \
                                 CAST_C(ori_kv), CAST_C(kv_bias), CAST_M(new_k), CAST_M(new_v), \
                                 (long)offset_per_layer, batch_seq_len, dim_per_head,          \
                                 head_num);                                                    \
  }
LSH_ENCDEC_KV(lsh_ker_arrange_encdec_kv_f16, __half, H, HM)
LSH_ENCDEC_KV(lsh_ker_arrange_encdec_kv_f32, float, F, FM)
#undef LSH_ENCDEC_KV

int lsh_ker_correlation_softmax_encdec_f16(int batch_size, int head_num_per_seq,
                                           int batch_seq_len, lsh_stream_t stream,
                                           void* correlation, const int* src_padding_mask) {
  return correlation_softmax_encdec<__half>(batch_size, head_num_per_seq, batch_seq_len,
                                            HS(stream), HM(correlation), src_padding_mask);
}
int lsh_ker_correlation_softmax_encdec_f32(int batch_size, int head_num_per_seq,
                                           int batch_seq_len, lsh_stream_t stream,
                                           void* correlation, const int* src_padding_mask) {
  return correlation_softmax_encdec<float>(batch_size, head_num_per_seq, batch_seq_len,
                                           HS(stream), FM(correlation), src_padding_mask);
}
int lsh_encdec_attention_f16(const void* q, const void* k, const void* v, const int* pad_mask,
                             void* ctx, int8_t* ctx_q, float quant_scale, int batch_size,
                             int beam_size, int head_num, int batch_seq_len, int dim_per_head,
                             lsh_stream_t stream) {
  return encdec_attention_f16(H(q), H(k), H(v), pad_mask, HM(ctx), ctx_q, quant_scale, batch_size,
                              beam_size, head_num, batch_seq_len, dim_per_head, HS(stream));
}
int lsh_gemm_f16_nt(const void* A, const void* W, void* C, int m, int n, int k,
                    lsh_stream_t stream) {
  return gemm_f16_nt(H(A), H(W), HM(C), m, n, k, HS(stream));
}

// ---- beam search -------------------------------------------------------------------
float lsh_length_norm(int length, float alpha) { return length_norm(length, alpha); }

#define LSH_SELECT_BEAM(NAME, TY, CAST_C)                                                      \
  int NAME(const int8_t* logits, const void* logit_bias, const float* seq_probs,               \
           const float* seq_score, const int* alive_seq, float dequant_scale, int* can_idx,    \
           float* can_score, int* num_beam_can, int vocab_size, int max_step,                  \
           float length_norm_v, int cur_step, int step_token_num, int max_thread_per_block,    \
           lsh_stream_t stream, int beam_size, float diverse_lambda, int end_id,               \
           int in_col32) {                                                                     \
    if (int rc = no_col32(in_col32, 0, "select_beam_rough_topk_i8I")) return rc;               \
    return select_beam_rough_topk_i8I<TY>(logits, CAST_C(logit_bias), seq_probs, seq_score,    \
                                          alive_seq, dequant_scale, can_idx, can_score,        \
                                          num_beam_can, vocab_size, max_step, length_norm_v,   \
                                          cur_step, step_token_num, max_thread_per_block,      \
                                          HS(stream), beam_size, diverse_lambda, end_id);      \
  }
LSH_SELECT_BEAM(lsh_select_beam_rough_topk_i8I_f16, __half, H)
LSH_SELECT_BEAM(lsh_select_beam_rough_topk_i8I_f32, float, F)
#undef LSH_SELECT_BEAM

int lsh_ker_refresh_result(const int* can_idx, const float* can_score,
                           const int* num_can_per_beam, const int* old_alive_seq,
                           int* new_alive_seq, float* seq_probs, float* seq_score,
                           int* num_finish_beam, int vocab_size, int cur_step,
                           float length_norm_v, float diverse_lambda, int end_id, int batch_size,
                           int beam_size, int max_step, lsh_stream_t stream) {
  return refresh_result(can_idx, can_score, num_can_per_beam, old_alive_seq, new_alive_seq,
                        seq_probs, seq_score, num_finish_beam, vocab_size, cur_step,
                        length_norm_v, diverse_lambda, end_id, batch_size, beam_size, max_step,
                        HS(stream));
}
int lsh_ker_refresh_cache_i8(int grid_dim_x, int grid_dim_y, int block_dim, lsh_stream_t stream,
                             const int* num_can_per_beam, const int* can_idx,
                             const int8_t* self_k_bgeem, const int8_t* self_v_bgeem,
                             int8_t* new_self_k_bgeem, int8_t* new_self_v_bgeem,
                             int64_t self_k_bgeem_offset, int beam_size, int dim_per_head,
                             int head_num, int vocab_size, int cur_step, int max_step,
                             int diverse, int end_id) {
  (void)block_dim;
  return refresh_cache_i8(grid_dim_x, grid_dim_y, HS(stream), num_can_per_beam, can_idx,
                          self_k_bgeem, self_v_bgeem, new_self_k_bgeem, new_self_v_bgeem,
                          (long)self_k_bgeem_offset, beam_size, dim_per_head, head_num,
                          vocab_size, cur_step, max_step, diverse != 0, end_id);
}
int lsh_ker_write_trg_tokenid_pos_penalty(const int* alive_seq, float* seq_score, int* output,
                                          int max_step, int beam_size, int batch_size,
                                          int out_len, lsh_stream_t stream) {
  return write_trg_tokenid_pos_penalty(alive_seq, seq_score, output, max_step, beam_size,
                                       batch_size, out_len, HS(stream));
}
int lsh_ker_write_trg_tokenid_neg_penalty(const int* alive_seq, const float* seq_score,
                                          int* output, int max_step, int beam_size,
                                          int vocab_size, int end_id, int batch_size, int out_len,
                                          lsh_stream_t stream) {
  return write_trg_tokenid_neg_penalty(alive_seq, seq_score, output, max_step, beam_size,
                                       vocab_size, end_id, batch_size, out_len, HS(stream));
}
int lsh_ker_write_topk_result(const int* alive_seq, float* seq_score, int* res_seq,
                              int vocab_size, int max_step, int beam_size, int end_id,
                              int batch_beam_num, int out_len, lsh_stream_t stream) {
  return write_topk_result(alive_seq, seq_score, res_seq, vocab_size, max_step, beam_size, end_id,
                           batch_beam_num, out_len, HS(stream));
}

#define LSH_BEAM_STEP(NAME, TY, CAST_C)                                                        \
  int NAME(const int8_t* logits, const void* logit_bias, float* seq_probs, float* seq_score,   \
           const int* old_alive_seq, int* new_alive_seq, float* top_score, int* top_idx,       \
           int* parent, int* num_finished, float dequant_scale, int vocab_size, int max_step,  \
           float length_norm_v, int cur_step, int batch_size, int beam_size, int end_id,       \
           lsh_stream_t stream) {                                                              \
    return beam_search_step_i8I<TY>(logits, CAST_C(logit_bias), seq_probs, seq_score,          \
                                    old_alive_seq, new_alive_seq, top_score, top_idx, parent,  \
                                    num_finished, dequant_scale, vocab_size, max_step,         \
                                    length_norm_v, cur_step, batch_size, beam_size, end_id,    \
                                    HS(stream));                                               \
  }
LSH_BEAM_STEP(lsh_beam_search_step_i8I_f16, __half, H)
LSH_BEAM_STEP(lsh_beam_search_step_i8I_f32, float, F)
#undef LSH_BEAM_STEP
int64_t lsh_beam_search_step_workspace(int batch_size, int beam_size, int vocab_size) {
  return (int64_t)beam_search_step_workspace_words(batch_size, beam_size, vocab_size) * 4;
}
#define LSH_BEAM_STEP_WS(NAME, TY, CAST_C)                                                     \
  int NAME(const int8_t* logits, const void* logit_bias, float* seq_probs, float* seq_score,   \
           const int* old_alive_seq, int* new_alive_seq, float* top_score, int* top_idx,       \
           int* parent, int* num_finished, float dequant_scale, int vocab_size, int max_step,  \
           float length_norm_v, int cur_step, int batch_size, int beam_size, int end_id,       \
           void* workspace, int64_t workspace_bytes, lsh_stream_t stream) {                    \
    if (workspace_bytes < 0) return lsh_fail(LSH_ERR_INVALID, #NAME ": negative workspace");   \
    return beam_search_step_i8I<TY>(logits, CAST_C(logit_bias), seq_probs, seq_score,          \
                                    old_alive_seq, new_alive_seq, top_score, top_idx, parent,  \
                                    num_finished, dequant_scale, vocab_size, max_step,         \
                                    length_norm_v, cur_step, batch_size, beam_size, end_id,    \
                                    HS(stream), static_cast<float*>(workspace),                \
                                    (size_t)workspace_bytes / 4);                              \
  }
LSH_BEAM_STEP_WS(lsh_beam_search_step_ws_i8I_f16, __half, H)
LSH_BEAM_STEP_WS(lsh_beam_search_step_ws_i8I_f32, float, F)
#undef LSH_BEAM_STEP_WS

int lsh_beam_search_step_noalloc_i8I_f16(const int8_t* logits, const void* logit_bias,
                                         float* seq_probs, float* seq_score,
                                         const int* old_alive_seq, int* new_alive_seq, int* parent,
                                         int* num_finished, float dequant_scale, int vocab_size,
                                         int max_step, float length_norm_v, int cur_step,
                                         int batch_size, int beam_size, int end_id,
                                         lsh_stream_t stream) {
  return beam_search_step_noalloc_i8I_f16(logits, H(logit_bias), seq_probs, seq_score,
                                          old_alive_seq, new_alive_seq, parent, num_finished,
                                          dequant_scale, vocab_size, max_step, length_norm_v,
                                          cur_step, batch_size, beam_size, end_id, HS(stream));
}

int lsh_refresh_cache_by_parent_i8(int n_layer, int rows, lsh_stream_t stream, const int* parent,
                                   const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                                   int8_t* v_new, int64_t layer_offset, int beam_size,
                                   int dim_per_head, int head_num, int cur_step, int max_step) {
  return refresh_cache_by_parent_i8(n_layer, rows, HS(stream), parent, k_old, v_old, k_new, v_new,
                                    (long)layer_offset, beam_size, dim_per_head, head_num,
                                    cur_step, max_step);
}

// ---- GPT path ------------------------------------------------------------------------
int lsh_ker_gpt_embedding_i8I_f16(int batch_size, int batch_seq_len, int hidden_size,
                                  lsh_stream_t stream, const int8_t* token_emb,
                                  const void* pos_emb, const int* token_id, void* output,
                                  int* real_seq_len, int padding_id, int pos_offset,
                                  float dequant_scale) {
  return gpt_embedding_i8I<__half>(batch_size, batch_seq_len, hidden_size, HS(stream), token_emb,
                                   H(pos_emb), token_id, HM(output), real_seq_len, padding_id,
                                   pos_offset, dequant_scale, 0, 0);
}
int lsh_ker_gpt_embedding_i8I_f32(int batch_size, int batch_seq_len, int hidden_size,
                                  lsh_stream_t stream, const int8_t* token_emb,
                                  const void* pos_emb, const int* token_id, void* output,
                                  int* real_seq_len, int padding_id, int pos_offset,
                                  float dequant_scale) {
  return gpt_embedding_i8I<float>(batch_size, batch_seq_len, hidden_size, HS(stream), token_emb,
                                  F(pos_emb), token_id, FM(output), real_seq_len, padding_id,
                                  pos_offset, dequant_scale, 0, 0);
}
int lsh_gpt_scores_i8_i32o(const int8_t* k, const int8_t* q, int32_t* scores, int batch_head_num,
                           int batch_seq_len, int dim_per_head, lsh_stream_t stream) {
  return gpt_scores_i8(q, k, scores, batch_head_num, batch_seq_len, dim_per_head, HS(stream));
}
int lsh_ker_correlation_softmax_gpt_i32I_f16(int batch_size, int batch_seq_len, int head_num,
                                             lsh_stream_t stream, const int32_t* correlation,
                                             void* output, const int* real_seq_len,
                                             float attn_scale, float dequant_scale) {
  return correlation_softmax_gpt_i32I<__half>(batch_size, batch_seq_len, head_num, HS(stream),
                                              correlation, HM(output), real_seq_len, attn_scale,
                                              dequant_scale);
}
int lsh_ker_correlation_softmax_gpt_i32I_f32(int batch_size, int batch_seq_len, int head_num,
                                             lsh_stream_t stream, const int32_t* correlation,
                                             void* output, const int* real_seq_len,
                                             float attn_scale, float dequant_scale) {
  return correlation_softmax_gpt_i32I<float>(batch_size, batch_seq_len, head_num, HS(stream),
                                             correlation, FM(output), real_seq_len, attn_scale,
                                             dequant_scale);
}
#define LSH_QKV_CACHE(NAME, TY, CAST_C)                                                        \
  int NAME(int batch_token_num, int hidden_size, lsh_stream_t stream, const int8_t* ori_qkv,   \
           const void* qkv_bias, int8_t* new_q, int8_t* new_k, const int8_t* k_cache,          \
           int8_t* new_v, const int8_t* v_cache, int batch_seq_len, int dim_per_head,          \
           int head_num, float dequant_scale, float quant_scale, int in_col32) {               \
    if (int rc = no_col32(in_col32, 0, "ker_arrange_qkv_with_cache_i8I_i8O")) return rc;       \
    return arrange_qkv_with_cache_i8I_i8O<TY>(batch_token_num, hidden_size, HS(stream),        \
                                              ori_qkv, CAST_C(qkv_bias), new_q, new_k, k_cache, \
                                              new_v, v_cache, batch_seq_len, dim_per_head,     \
                                              head_num, dequant_scale, quant_scale);           \
  }
LSH_QKV_CACHE(lsh_ker_arrange_qkv_with_cache_i8I_i8O_f16, __half, H)
LSH_QKV_CACHE(lsh_ker_arrange_qkv_with_cache_i8I_i8O_f32, float, F)
#undef LSH_QKV_CACHE

int lsh_ker_topk_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len,
                            int max_thread_per_block, lsh_stream_t stream, const int8_t* logits,
                            int* old_input_ids, int* new_input_ids, const int* real_seq_len,
                            int vocab_size, int k, int* unfinished, void* curandstate, int eos_id,
                            float dequant_scale, int in_col32) {
  (void)max_thread_per_block;
  (void)real_seq_len;
  if (int rc = no_col32(in_col32, 0, "ker_topk_sample_i8I")) return rc;
  if (!(dequant_scale > 0.f))
    return lsh_fail(LSH_ERR_INVALID, "ker_topk_sample_i8I: dequant_scale must be positive");
  return topk_sample_i8I(batch_size, batch_seq_len, logits_seq_len, HS(stream), logits,
                         old_input_ids, new_input_ids, vocab_size, k, unfinished, eos_id,
                         curandstate, dequant_scale);
}
int lsh_ker_topp_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len,
                            int max_thread_per_block, lsh_stream_t stream, const int8_t* logits,
                            int* old_input_ids, int* new_input_ids, const int* real_seq_len,
                            int vocab_size, float p, int* unfinished, void* curandstate,
                            int eos_id, float dequant_scale, int in_col32) {
  (void)max_thread_per_block;
  (void)real_seq_len;
  if (int rc = no_col32(in_col32, 0, "ker_topp_sample_i8I")) return rc;
  return topp_sample_i8I(batch_size, batch_seq_len, logits_seq_len, HS(stream), logits,
                         old_input_ids, new_input_ids, vocab_size, p, unfinished, curandstate,
                         eos_id, dequant_scale);
}
#define LSH_DEC_SAMPLE(SUF, T)                                                                  \
  int lsh_ker_topk_sample_i8I_dec_##SUF(                                                        \
      int batch_size, int batch_seq_len, int max_step, int logits_seq_len,                      \
      int max_thread_per_block, lsh_stream_t stream, const int8_t* logits,                      \
      const void* logit_bias, int* old_input_ids, int* new_input_ids, int vocab_size, int k,    \
      int* all_finished, void* curandstate, int eos_id, float dequant_scale, int in_col32) {    \
    (void)max_thread_per_block;                                                                 \
    (void)new_input_ids;                                                                        \
    if (int rc = no_col32(in_col32, 0, "ker_topk_sample_i8I")) return rc;                       \
    return dec_topk_sample_i8I<T>(batch_size, batch_seq_len, max_step, logits_seq_len,          \
                                  HS(stream), logits, static_cast<const T*>(logit_bias),        \
                                  old_input_ids, vocab_size, k, all_finished, curandstate,      \
                                  eos_id, dequant_scale);                                       \
  }                                                                                             \
  int lsh_ker_topp_sample_i8I_dec_##SUF(                                                        \
      int batch_size, int batch_seq_len, int max_step, int logits_seq_len,                      \
      int max_thread_per_block, lsh_stream_t stream, const int8_t* logits,                      \
      const void* logit_bias, int* old_input_ids, int* new_input_ids, int vocab_size, float p,  \
      int* unfinished, void* curandstate, int eos_id, float dequant_scale, int in_col32) {      \
    (void)max_thread_per_block;                                                                 \
    (void)new_input_ids;                                                                        \
    if (int rc = no_col32(in_col32, 0, "ker_topp_sample_i8I")) return rc;                       \
    return dec_topp_sample_i8I<T>(batch_size, batch_seq_len, max_step, logits_seq_len,          \
                                  HS(stream), logits, static_cast<const T*>(logit_bias),        \
                                  old_input_ids, vocab_size, p, unfinished, curandstate,        \
                                  eos_id, dequant_scale);                                       \
  }                                                                                             \
  int lsh_ker_attention_mask_weights_i32I_##SUF(                                                \
      int batch_size, int dst_seq_len, int src_seq_len, int head_num, lsh_stream_t stream,      \
      const int32_t* correlation, void* output, const int* real_seq_len, float attn_scale,      \
      float dequant_scale) {                                                                    \
    return attention_mask_weights_i32I<T>(batch_size, dst_seq_len, src_seq_len, head_num,       \
                                          HS(stream), correlation, static_cast<T*>(output),     \
                                          real_seq_len, attn_scale, dequant_scale);             \
  }
LSH_DEC_SAMPLE(f16, __half)
LSH_DEC_SAMPLE(f32, float)
#undef LSH_DEC_SAMPLE

int lsh_rng_setup(void* state, int n, uint64_t seed, lsh_stream_t stream) {
  return sample_state_setup(state, n, seed, HS(stream));
}
int lsh_ker_ppl_i8I(int batch_size, int batch_seq_len, int max_thread_per_block,
                    lsh_stream_t stream, const int8_t* logits, const int* input_ids,
                    const int* real_seq_len, float* ppl, int vocab_size, float dequant_scale,
                    int in_col32) {
  (void)max_thread_per_block;
  if (int rc = no_col32(in_col32, 0, "ker_ppl_i8I")) return rc;
  return ppl_i8I(batch_size, batch_seq_len, HS(stream), logits, input_ids, real_seq_len, ppl,
                 vocab_size, dequant_scale);
}
int lsh_ker_ppl_i8I_workspace(int batch_size, int batch_seq_len, lsh_stream_t stream,
                              const int8_t* logits, const int* input_ids, const int* real_seq_len,
                              float* ppl, int vocab_size, float dequant_scale, float* workspace) {
  if (!workspace) return lsh_fail(LSH_ERR_INVALID, "ker_ppl_i8I: null workspace");
  return ppl_i8I(batch_size, batch_seq_len, HS(stream), logits, input_ids, real_seq_len, ppl,
                 vocab_size, dequant_scale, workspace);
}
int lsh_gpt_arrange_qkv_prefill_f16(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                    const int8_t* ori_qkv, const void* qkv_bias, void* q_codes,
                                    void* k_codes, void* v_deq, int8_t* k_cache, int8_t* v_cache,
                                    int batch_seq_len, int dim_per_head, int head_num,
                                    int max_step, float dequant_scale, float quant_scale) {
  return gpt_arrange_qkv_prefill_f16(batch_token_num, hidden_size, HS(stream), ori_qkv,
                                     H(qkv_bias), HM(q_codes), HM(k_codes), HM(v_deq), k_cache,
                                     v_cache, batch_seq_len, dim_per_head, head_num, max_step,
                                     dequant_scale, quant_scale);
}
int lsh_gpt_prefill_attention_f16(const void* q_codes, const void* k_codes, const void* v,
                                  const int* real_seq_len, void* ctx, int8_t* ctx_q,
                                  float quant_scale, float dequant_scale, int batch_size,
                                  int batch_seq_len, int head_num, int dim_per_head,
                                  lsh_stream_t stream) {
  return gpt_prefill_attention_f16(H(q_codes), H(k_codes), H(v), real_seq_len, HM(ctx), ctx_q,
                                   quant_scale, dequant_scale, batch_size, batch_seq_len,
                                   head_num, dim_per_head, HS(stream));
}
int lsh_gpt_prefill_on_codes_in_models(int on) { return gpt_prefill_i8_enable(on != 0) ? 1 : 0; }
int lsh_gpt_prefill_i8_supported(int batch_seq_len, int head_num, int dim_per_head) {
  return gpt_prefill_i8_supported(batch_seq_len, head_num, dim_per_head) ? 1 : 0;
}
int lsh_gpt_arrange_qkv_prefill_i8(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                   const int8_t* ori_qkv, const void* qkv_bias, int8_t* q_codes,
                                   int8_t* k_cache, int8_t* v_cache, int batch_seq_len,
                                   int dim_per_head, int head_num, int max_step,
                                   float dequant_scale, float quant_scale) {
  return gpt_arrange_qkv_prefill_i8(batch_token_num, hidden_size, HS(stream), ori_qkv, H(qkv_bias),
                                    q_codes, k_cache, v_cache, batch_seq_len, dim_per_head,
                                    head_num, max_step, dequant_scale, quant_scale);
}
int lsh_gpt_prefill_attention_i8(const int8_t* q_codes, const int8_t* k_cache,
                                 const int8_t* v_cache, const int* real_seq_len, int8_t* ctx_q,
                                 float quant_scale, float dequant_scale, float v_quant_scale,
                                 int batch_size, int batch_seq_len, int head_num, int dim_per_head,
                                 int max_step, lsh_stream_t stream) {
  return gpt_prefill_attention_i8(q_codes, k_cache, v_cache, real_seq_len, ctx_q, quant_scale,
                                  dequant_scale, v_quant_scale, batch_size, batch_seq_len, head_num,
                                  dim_per_head, max_step, HS(stream));
}
int lsh_gpt_greedy_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size,
                        int max_step, int cur_len, int batch_size, int* unfinished, int eos_id,
                        lsh_stream_t stream) {
  return gpt_greedy_step(logits, ids, last_ids, vocab_size, max_step, cur_len, batch_size,
                         unfinished, eos_id, HS(stream));
}
int lsh_gpt_sample_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size,
                        int max_step, int cur_len, int batch_size, int* unfinished, int eos_id,
                        int k, float p, float dequant_scale, void* state, lsh_stream_t stream) {
  return gpt_sample_step(logits, ids, last_ids, vocab_size, max_step, cur_len, batch_size,
                         unfinished, eos_id, k, p, dequant_scale, state, HS(stream));
}

}  // extern "C"
