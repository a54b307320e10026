// extern "C" surface of the operator launchers declared in include/lightseq_ops.h:
// argument checks that need no kernel knowledge and the dispatch on the storage type.
#include "ls_launch.h"
#include "../../include/lightseq_ops.h"

using namespace lsh;

namespace {

int no_col32(int flag, const char* who) {
  if (!flag) return LSH_OK;
  static thread_local std::string msg;
  msg = std::string(who) + ": COL32 layouts are cuBLASLt-specific and not provided";
  return lsh_fail(LSH_ERR_UNSUPPORTED, msg.c_str());
}

template <typename T>
const T* C(const void* p) { return reinterpret_cast<const T*>(p); }
template <typename T>
T* M(void* p) { return reinterpret_cast<T*>(p); }
hipStream_t HS(lsh_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace

// Expands BODY once with T = __half / suffix _f16 and once with T = float / suffix _f32.
#define LSH_BOTH(NAME, PARAMS, ...)                         \
  int NAME##_f16 PARAMS { typedef __half T; __VA_ARGS__ }   \
  int NAME##_f32 PARAMS { typedef float T; __VA_ARGS__ }

extern "C" {

LSH_BOTH(lsh_launch_quantize,
         (int8_t* q_ptr, uint8_t* clip_mask_ptr, float* alpha_ptr, const void* f_ptr,
          const void* clip_max_ptr, int numel, int mask_start_bit, lsh_stream_t stream),
         return opb_quantize<T>(q_ptr, clip_mask_ptr, alpha_ptr, C<T>(f_ptr), C<T>(clip_max_ptr),
                                numel, 1, mask_start_bit, HS(stream));)

LSH_BOTH(lsh_launch_quantize_2d,
         (int8_t* q_ptr, uint8_t* clip_mask_ptr, float* alpha_ptr, const void* f_ptr,
          const void* clip_max_ptr, int batch_tokens, int hidden_size, int mask_start_bit,
          lsh_stream_t stream, int out_layout),
         if (out_layout != 0)
           return lsh_fail(LSH_ERR_UNSUPPORTED,
                           "launch_quantize: only the row-major output layout is provided");
         if (batch_tokens <= 0 || hidden_size <= 0)
           return lsh_fail(LSH_ERR_INVALID, "launch_quantize: bad shape");
         return opb_quantize<T>(q_ptr, clip_mask_ptr, alpha_ptr, C<T>(f_ptr), C<T>(clip_max_ptr),
                                (long)batch_tokens * hidden_size, batch_tokens, mask_start_bit,
                                HS(stream));)

LSH_BOTH(lsh_launch_fake_quantize,
         (uint8_t* clip_mask_ptr, float* alpha_ptr, void* output, const void* input,
          const void* clip_max_ptr, int numel, int mask_start_bit, lsh_stream_t stream,
          int symmetry),
         return opb_fake_quantize<T>(clip_mask_ptr, alpha_ptr, M<T>(output), C<T>(input),
                                     C<T>(clip_max_ptr), numel, mask_start_bit, symmetry != 0,
                                     HS(stream));)

LSH_BOTH(lsh_launch_dequantize,
         (void* f_ptr, const int8_t* q_ptr, const void* clip_max_ptr, int numel,
          int mask_start_bit, lsh_stream_t stream),
         (void)mask_start_bit;
         return opb_dequantize<T>(M<T>(f_ptr), q_ptr, C<T>(clip_max_ptr), numel, HS(stream));)

LSH_BOTH(lsh_launch_layer_norm,
         (void* ln_res, void* vars, void* means, const void* inp, const void* scale,
          const void* bias, int batch_size, int hidden_dim, lsh_stream_t stream),
         if (!ln_res) return lsh_fail(LSH_ERR_INVALID, "launch_layer_norm: null output");
         return opb_layer_norm<T>(M<T>(ln_res), nullptr, nullptr, M<T>(vars), M<T>(means),
                                  C<T>(inp), C<T>(scale), C<T>(bias), nullptr, batch_size,
                                  hidden_dim, HS(stream));)

LSH_BOTH(lsh_launch_layer_norm_i8,
         (int8_t* q_out, uint8_t* clip_mask_out, void* vars, void* means, const void* inp,
          const void* gamma, const void* betta, const void* clip_max_out, int batch_size,
          int hidden_dim, lsh_stream_t stream),
         if (!q_out) return lsh_fail(LSH_ERR_INVALID, "launch_layer_norm_i8: null output");
         return opb_layer_norm<T>(nullptr, q_out, clip_mask_out, M<T>(vars), M<T>(means),
                                  C<T>(inp), C<T>(gamma), C<T>(betta), C<T>(clip_max_out),
                                  batch_size, hidden_dim, HS(stream));)

LSH_BOTH(lsh_launch_attn_softmax,
         (void* vals, const void* attn_mask, int batch_size, int heads, int from_len, int to_len,
          int mask_future, lsh_stream_t stream),
         return opb_attn_softmax<T>(M<T>(vals), C<T>(attn_mask), batch_size, heads, from_len,
                                    to_len, mask_future != 0, HS(stream));)

LSH_BOTH(lsh_launch_quant_bias_add_transform_20314,
         (void* output, uint8_t* clip_mask, const int8_t* input, const void* bias,
          const void* clip_max, int dim_0, int dim_1, int dim_2, int dim_3, int dim_4,
          lsh_stream_t stream, const void* out_clip_max, int in_col32),
         if (int rc = no_col32(in_col32, "launch_quant_bias_add_transform_20314")) return rc;
         return opb_quant_bias_add_transform_20314<T>(M<T>(output), clip_mask, input, C<T>(bias),
                                                      C<T>(clip_max), dim_0, dim_1, dim_2, dim_3,
                                                      dim_4, HS(stream), C<T>(out_clip_max));)

LSH_BOTH(lsh_launch_bias_add_transform_20314,
         (void* output, const void* input, const void* bias, int dim_0, int dim_1, int dim_2,
          int dim_3, int dim_4, lsh_stream_t stream),
         return opb_bias_add_transform_20314<T>(M<T>(output), C<T>(input), C<T>(bias), dim_0,
                                                dim_1, dim_2, dim_3, dim_4, HS(stream));)

LSH_BOTH(lsh_launch_concat3_dim1,
         (const void* inp1, const void* inp2, void* output, int sz0, int sz2, int sz1_1,
          int sz1_2, lsh_stream_t stream),
         return opb_concat3_dim1<T>(C<T>(inp1), C<T>(inp2), M<T>(output), sz0, sz2, sz1_1, sz1_2,
                                    HS(stream));)

LSH_BOTH(lsh_launch_transform4d_0213,
         (void* output, const void* vals, int batch_size, int seq_len, int hidden_dim, int nhead,
          int trans_count, lsh_stream_t stream),
         if (!output) return lsh_fail(LSH_ERR_INVALID, "launch_transform4d_0213: null output");
         return opb_transform4d_0213<T>(M<T>(output), nullptr, nullptr, C<T>(vals), nullptr,
                                        batch_size, seq_len, hidden_dim, nhead, trans_count,
                                        HS(stream));)

LSH_BOTH(lsh_launch_quant_transform4d_0213,
         (int8_t* output, uint8_t* clip_mask, const void* vals, const void* clip_max,
          int batch_size, int seq_len, int hidden_dim, int nhead, int trans_count,
          lsh_stream_t stream),
         if (!output)
           return lsh_fail(LSH_ERR_INVALID, "launch_quant_transform4d_0213: null output");
         return opb_transform4d_0213<T>(nullptr, output, clip_mask, C<T>(vals), C<T>(clip_max),
                                        batch_size, seq_len, hidden_dim, nhead, trans_count,
                                        HS(stream));)

LSH_BOTH(lsh_launch_ls_dropout,
         (void* out, const void* vals, uint8_t* mask, int total_count, float ratio,
          lsh_stream_t stream, int backward),
         if (backward)
           return lsh_fail(LSH_ERR_UNSUPPORTED, "launch_ls_dropout: backward is not provided");
         return opb_dropout<T>(M<T>(out), C<T>(vals), mask, total_count, ratio, HS(stream));)

LSH_BOTH(lsh_launch_ls_dropout_res_bias,
         (void* out, const void* vals, uint8_t* mask, const void* bias, const void* residual,
          int total_count, int dim, float ratio, lsh_stream_t stream),
         return opb_dropout_res_bias<T>(M<T>(out), C<T>(vals), mask, C<T>(bias), C<T>(residual),
                                        total_count, dim, ratio, HS(stream));)

#define LSH_ACT_BIAS(ACTNAME, ACT)                                                              \
  LSH_BOTH(lsh_launch_ls_dropout_act_bias_##ACTNAME,                                            \
           (void* out, const void* vals, uint8_t* mask, const void* bias, int total_count,      \
            int dim, float ratio, lsh_stream_t stream),                                         \
           return opb_dropout_act_bias<T>(ACT, M<T>(out), C<T>(vals), mask, C<T>(bias),         \
                                          total_count, dim, ratio, HS(stream));)                \
  LSH_BOTH(lsh_launch_ls_quant_dropout_act_bias_##ACTNAME,                                      \
           (int8_t* qout, uint8_t* cmask_out, uint8_t* cmask_in, uint8_t* dropout_mask,         \
            const int8_t* qinput, const void* bias, const void* cmax_out, const void* cmax_in,  \
            int total_count, int dim, float ratio, lsh_stream_t stream),                        \
           if (!qout) return lsh_fail(LSH_ERR_INVALID,                                          \
                                      "launch_ls_quant_dropout_act_bias: null output");         \
           return opb_quant_dropout_act_bias<T>(ACT, qout, nullptr, cmask_out, cmask_in,        \
                                                dropout_mask, qinput, C<T>(bias),               \
                                                C<T>(cmax_out), C<T>(cmax_in), total_count,     \
                                                dim, ratio, true, HS(stream));)                 \
  LSH_BOTH(lsh_launch_ls_fakequant_dropout_act_bias_##ACTNAME,                                  \
           (void* out, uint8_t* cmask_out, uint8_t* cmask_in, uint8_t* dropout_mask,            \
            const int8_t* qinput, const void* bias, const void* cmax_out, const void* cmax_in,  \
            int total_count, int dim, float ratio, lsh_stream_t stream, int in_col32,           \
            int symmetry),                                                                      \
           if (int rc = no_col32(in_col32, "launch_ls_fakequant_dropout_act_bias")) return rc;  \
           if (!out) return lsh_fail(LSH_ERR_INVALID,                                           \
                                     "launch_ls_fakequant_dropout_act_bias: null output");      \
           return opb_quant_dropout_act_bias<T>(ACT, nullptr, M<T>(out), cmask_out, cmask_in,   \
                                                dropout_mask, qinput, C<T>(bias),               \
                                                C<T>(cmax_out), C<T>(cmax_in), total_count,     \
                                                dim, ratio, symmetry != 0, HS(stream));)
LSH_ACT_BIAS(gelu, 0)
LSH_ACT_BIAS(relu, 1)
#undef LSH_ACT_BIAS

LSH_BOTH(lsh_launch_ls_quant_dropout_res_bias,
         (void* out, uint8_t* mask, const int8_t* qvals, const void* cmax, const void* bias,
          const void* residual, int total_count, int dim, float ratio, lsh_stream_t stream,
          int in_col32),
         if (int rc = no_col32(in_col32, "launch_ls_quant_dropout_res_bias")) return rc;
         return opb_quant_dropout_res_bias<T>(M<T>(out), mask, qvals, C<T>(cmax), C<T>(bias),
                                              C<T>(residual), total_count, dim, ratio,
                                              HS(stream));)

int lsh_feed_forward_i8(int bsz, int output_size, int input_size, const int8_t* qinput_ptr,
                        const int8_t* qweight_ptr, const float* alpha_ptr, const float* beta_ptr,
                        int8_t* qout_ptr, lsh_stream_t stream) {
  (void)beta_ptr;  // the layers keep a device 0.0 there (transformer_encoder_layer.h:211-212)
  return gemm_i8_i8o_dev_alpha(qinput_ptr, qweight_ptr, qout_ptr, bsz, output_size, input_size,
                               alpha_ptr, HS(stream));
}

int lsh_layer_attention_f16(const void* q, const void* k, const void* v, const void* attn_mask,
                            void* ctx, int batch_size, int seq_len, int heads, int dim_per_head,
                            int mask_future, lsh_stream_t stream) {
  return layer_attention_f16(C<__half>(q), C<__half>(k), C<__half>(v), C<__half>(attn_mask),
                             M<__half>(ctx), batch_size, seq_len, heads, dim_per_head,
                             mask_future != 0, HS(stream));
}

LSH_BOTH(lsh_strided_batch_gemm,
         (int bsz, int m, int n, int k, float alpha, float beta, int op_a, int op_b,
          const void* buffer_a, const void* buffer_b, void* output, lsh_stream_t stream),
         return strided_batch_gemm<T>(bsz, m, n, k, alpha, beta, op_a, op_b, C<T>(buffer_a),
                                      C<T>(buffer_b), M<T>(output), HS(stream));)

int lsh_layer_cross_attention_f16(const void* q, const void* k, const void* v,
                                  const void* attn_mask, void* ctx, int batch_size, int from_len,
                                  int to_len, int heads, int dim_per_head, int mask_future,
                                  lsh_stream_t stream) {
  return layer_cross_attention_f16(C<__half>(q), C<__half>(k), C<__half>(v), C<__half>(attn_mask),
                                   M<__half>(ctx), batch_size, from_len, to_len, heads,
                                   dim_per_head, mask_future != 0, HS(stream));
}

}  // extern "C"
