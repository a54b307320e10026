// extern "C" surface of the library: argument validation, status/error plumbing and
// dispatch on the storage type.  No kernel code lives here.
#include <string>

#include "ls_device.cuh"
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

// ---- LayerNorm family --------------------------------------------------------------
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

// ---- embedding ----------------------------------------------------------------------------------
int lsh_launch_enc_emb_i8I_f16(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               void* output, int* pad_mask, int pad_id, int batch_size,
                               int seq_len, int hidden_dim, lsh_stream_t stream,
                               const void* /*lang_emb*/, const int* /*lang_id*/, int multilg_type,
                               float dequant_scale, int scaled) {
  if (multilg_type != 0) return lsh_fail(LSH_ERR_INVALID, "multilingle not supported");
  return enc_emb_i8I<__half>(token_emb, H(pos_emb), tokens, HM(output), pad_mask, pad_id,
                             batch_size, seq_len, hidden_dim, HS(stream), dequant_scale,
                             scaled != 0);
}
int lsh_launch_enc_emb_i8I_f32(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               void* output, int* pad_mask, int pad_id, int batch_size,
                               int seq_len, int hidden_dim, lsh_stream_t stream,
                               const void* /*lang_emb*/, const int* /*lang_id*/, int multilg_type,
                               float dequant_scale, int scaled) {
  if (multilg_type != 0) return lsh_fail(LSH_ERR_INVALID, "multilingle not supported");
  return enc_emb_i8I<float>(token_emb, F(pos_emb), tokens, FM(output), pad_mask, pad_id,
                            batch_size, seq_len, hidden_dim, HS(stream), dequant_scale,
                            scaled != 0);
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

}  // extern "C"
