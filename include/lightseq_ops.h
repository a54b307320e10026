/*
 * lightseq_ops.h -- C ABI of the operator and layer interface of the quantised layer path
 * (the reference's lightseq/csrc tree: kernels/cuda/includes/kernels.h, the headers of
 * ops/includes and layers/includes, pybind/pybind_layer.cpp), forward only, one MI355X.
 *
 * Launchers keep the reference's names and argument order; the template parameter T
 * becomes the suffix _f16 / _f32, cudaStream_t becomes lsh_stream_t.  Clip values
 * ("clip_max", "cmax") are DEVICE pointers to T scalars, as in the reference, where they
 * live inside the layer's parameter blob.  Mask outputs (clip masks for the backward pass,
 * dropout masks) may be null.  Dropout ratios must be 0: cuRAND's Philox stream cannot be
 * reproduced and training is outside this library; any other ratio returns
 * LSH_ERR_UNSUPPORTED.  The cuBLASLt-specific output layouts of launch_quantize
 * (kCol32, kCOL4_4R2_8C, kCOL32_2R_4R4) and the in_col32 flags do not exist here.
 * Status codes and lsh_last_error() are those of lightseq_hip.h.
 */
#ifndef LIGHTSEQ_OPS_H_
#define LIGHTSEQ_OPS_H_

#include "lightseq_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- quantize / fake_quantize / dequantize -------------------------------------- */
/* kernels.h:232-235 launch_quantize (quantize_kernels.cu:41-149): q = quantize(f,
 * clip_max[0]); clip_mask |= mask bits at mask_start_bit; alpha (may be null) receives
 * clip_max[0] * clip_max[1] / (clip_max[2] * 127). */
int lsh_launch_quantize_f16(int8_t* q_ptr, uint8_t* clip_mask_ptr, float* alpha_ptr,
                            const void* f_ptr, const void* clip_max_ptr, int numel,
                            int mask_start_bit, lsh_stream_t stream);
int lsh_launch_quantize_f32(int8_t* q_ptr, uint8_t* clip_mask_ptr, float* alpha_ptr,
                            const void* f_ptr, const void* clip_max_ptr, int numel,
                            int mask_start_bit, lsh_stream_t stream);
/* kernels.h:237-241 (quantize_kernels.cu:600-758): the [batch_tokens, hidden_size] form;
 * alpha_ptr receives batch_tokens copies of alpha.  out_layout must be 0 (kRowMajor). */
int lsh_launch_quantize_2d_f16(int8_t* q_ptr, uint8_t* clip_mask_ptr, float* alpha_ptr,
                               const void* f_ptr, const void* clip_max_ptr, int batch_tokens,
                               int hidden_size, int mask_start_bit, lsh_stream_t stream,
                               int out_layout);
int lsh_launch_quantize_2d_f32(int8_t* q_ptr, uint8_t* clip_mask_ptr, float* alpha_ptr,
                               const void* f_ptr, const void* clip_max_ptr, int batch_tokens,
                               int hidden_size, int mask_start_bit, lsh_stream_t stream,
                               int out_layout);
/* kernels.h:243-247 launch_fake_quantize (quantize_kernels.cu:151-273) */
int lsh_launch_fake_quantize_f16(uint8_t* clip_mask_ptr, float* alpha_ptr, void* output,
                                 const void* input, const void* clip_max_ptr, int numel,
                                 int mask_start_bit, lsh_stream_t stream, int symmetry);
int lsh_launch_fake_quantize_f32(uint8_t* clip_mask_ptr, float* alpha_ptr, void* output,
                                 const void* input, const void* clip_max_ptr, int numel,
                                 int mask_start_bit, lsh_stream_t stream, int symmetry);
/* kernels.h:249-251 launch_dequantize (quantize_kernels.cu:275-348) */
int lsh_launch_dequantize_f16(void* f_ptr, const int8_t* q_ptr, const void* clip_max_ptr,
                              int numel, int mask_start_bit, lsh_stream_t stream);
int lsh_launch_dequantize_f32(void* f_ptr, const int8_t* q_ptr, const void* clip_max_ptr,
                              int numel, int mask_start_bit, lsh_stream_t stream);

/* ---- layer norm --------------------------------------------------------------------- */
/* kernels.h:24-27 launch_layer_norm (normalize_kernels.cu:40-180): vars receives
 * E[x^2] - E[x]^2 + 1e-8 per row, means (may be null) the mean. */
int lsh_launch_layer_norm_f16(void* ln_res, void* vars, void* means, const void* inp,
                              const void* scale, const void* bias, int batch_size,
                              int hidden_dim, lsh_stream_t stream);
int lsh_launch_layer_norm_f32(void* ln_res, void* vars, void* means, const void* inp,
                              const void* scale, const void* bias, int batch_size,
                              int hidden_dim, lsh_stream_t stream);
/* kernels.h:29-33 launch_layer_norm_i8 (normalize_kernels.cu:204-380) */
int lsh_launch_layer_norm_i8_f16(int8_t* q_out, uint8_t* clip_mask_out, void* vars, void* means,
                                 const void* inp, const void* gamma, const void* betta,
                                 const void* clip_max_out, int batch_size, int hidden_dim,
                                 lsh_stream_t stream);
int lsh_launch_layer_norm_i8_f32(int8_t* q_out, uint8_t* clip_mask_out, void* vars, void* means,
                                 const void* inp, const void* gamma, const void* betta,
                                 const void* clip_max_out, int batch_size, int hidden_dim,
                                 lsh_stream_t stream);

/* ---- attention softmax ---------------------------------------------------------------- */
/* kernels.h:47-50 launch_attn_softmax (softmax_kernels.cu:35-279): in place on
 * [batch, heads, from_len, to_len]; attn_mask [batch, to_len] additive, may be null. */
int lsh_launch_attn_softmax_f16(void* vals, const void* attn_mask, int batch_size, int heads,
                                int from_len, int to_len, int mask_future, lsh_stream_t stream);
int lsh_launch_attn_softmax_f32(void* vals, const void* attn_mask, int batch_size, int heads,
                                int from_len, int to_len, int mask_future, lsh_stream_t stream);

/* ---- head split / merge ------------------------------------------------------------------ */
/* kernels.h:85-93 launch_quant_bias_add_transform_20314 (transform_kernels.cu:253-424) */
int lsh_launch_quant_bias_add_transform_20314_f16(void* output, uint8_t* clip_mask,
                                                  const int8_t* input, const void* bias,
                                                  const void* clip_max, int dim_0, int dim_1,
                                                  int dim_2, int dim_3, int dim_4,
                                                  lsh_stream_t stream, const void* out_clip_max,
                                                  int in_col32);
int lsh_launch_quant_bias_add_transform_20314_f32(void* output, uint8_t* clip_mask,
                                                  const int8_t* input, const void* bias,
                                                  const void* clip_max, int dim_0, int dim_1,
                                                  int dim_2, int dim_3, int dim_4,
                                                  lsh_stream_t stream, const void* out_clip_max,
                                                  int in_col32);
/* kernels.h:72-75 launch_bias_add_transform_20314 (transform_kernels.cu:140-235): input
 * [dim_0, dim_1, dim_2, dim_3, dim_4] + bias [dim_2, dim_3, dim_4] -> [dim_2, dim_0, dim_3,
 * dim_1, dim_4] */
int lsh_launch_bias_add_transform_20314_f16(void* output, const void* input, const void* bias,
                                            int dim_0, int dim_1, int dim_2, int dim_3, int dim_4,
                                            lsh_stream_t stream);
int lsh_launch_bias_add_transform_20314_f32(void* output, const void* input, const void* bias,
                                            int dim_0, int dim_1, int dim_2, int dim_3, int dim_4,
                                            lsh_stream_t stream);
/* kernels.h:183-185 launch_concat3_dim1 (general_kernels.cu:187-234): inp1 [sz0, sz1_1, sz2]
 * and inp2 [sz0, sz1_2, sz2] joined along dimension 1; inp1 may be null when sz1_1 is 0 */
int lsh_launch_concat3_dim1_f16(const void* inp1, const void* inp2, void* output, int sz0, int sz2,
                                int sz1_1, int sz1_2, lsh_stream_t stream);
int lsh_launch_concat3_dim1_f32(const void* inp1, const void* inp2, void* output, int sz0, int sz2,
                                int sz1_1, int sz1_2, lsh_stream_t stream);
/* kernels.h:95-98 launch_transform4d_0213 (transform_kernels.cu:444-560) */
int lsh_launch_transform4d_0213_f16(void* output, const void* vals, int batch_size, int seq_len,
                                    int hidden_dim, int nhead, int trans_count,
                                    lsh_stream_t stream);
int lsh_launch_transform4d_0213_f32(void* output, const void* vals, int batch_size, int seq_len,
                                    int hidden_dim, int nhead, int trans_count,
                                    lsh_stream_t stream);
/* kernels.h:100-104 launch_quant_transform4d_0213 (transform_kernels.cu:567-680) */
int lsh_launch_quant_transform4d_0213_f16(int8_t* output, uint8_t* clip_mask, const void* vals,
                                          const void* clip_max, int batch_size, int seq_len,
                                          int hidden_dim, int nhead, int trans_count,
                                          lsh_stream_t stream);
int lsh_launch_quant_transform4d_0213_f32(int8_t* output, uint8_t* clip_mask, const void* vals,
                                          const void* clip_max, int batch_size, int seq_len,
                                          int hidden_dim, int nhead, int trans_count,
                                          lsh_stream_t stream);

/* ---- bias / activation / residual epilogues (dropout ratio 0) ------------------------------- */
/* kernels.h:112-114 launch_ls_dropout (forward; `backward` must be 0) */
int lsh_launch_ls_dropout_f16(void* out, const void* vals, uint8_t* mask, int total_count,
                              float ratio, lsh_stream_t stream, int backward);
int lsh_launch_ls_dropout_f32(void* out, const void* vals, uint8_t* mask, int total_count,
                              float ratio, lsh_stream_t stream, int backward);
/* kernels.h:116-120 launch_ls_dropout_res_bias (dropout_kernels.cu:373-505) */
int lsh_launch_ls_dropout_res_bias_f16(void* out, const void* vals, uint8_t* mask,
                                       const void* bias, const void* residual, int total_count,
                                       int dim, float ratio, lsh_stream_t stream);
int lsh_launch_ls_dropout_res_bias_f32(void* out, const void* vals, uint8_t* mask,
                                       const void* bias, const void* residual, int total_count,
                                       int dim, float ratio, lsh_stream_t stream);
/* kernels.h:122-125 launch_ls_dropout_act_bias<act> (dropout_kernels.cu:690-860) */
int lsh_launch_ls_dropout_act_bias_gelu_f16(void* out, const void* vals, uint8_t* mask,
                                            const void* bias, int total_count, int dim,
                                            float ratio, lsh_stream_t stream);
int lsh_launch_ls_dropout_act_bias_gelu_f32(void* out, const void* vals, uint8_t* mask,
                                            const void* bias, int total_count, int dim,
                                            float ratio, lsh_stream_t stream);
int lsh_launch_ls_dropout_act_bias_relu_f16(void* out, const void* vals, uint8_t* mask,
                                            const void* bias, int total_count, int dim,
                                            float ratio, lsh_stream_t stream);
int lsh_launch_ls_dropout_act_bias_relu_f32(void* out, const void* vals, uint8_t* mask,
                                            const void* bias, int total_count, int dim,
                                            float ratio, lsh_stream_t stream);
/* kernels.h:138-144 launch_ls_quant_dropout_act_bias<act> (dropout_kernels.cu:856-1057):
 * cmax_out dequantises qinput, cmax_in quantises the result. */
int lsh_launch_ls_quant_dropout_act_bias_gelu_f16(int8_t* qout, uint8_t* cmask_out,
                                                  uint8_t* cmask_in, uint8_t* dropout_mask,
                                                  const int8_t* qinput, const void* bias,
                                                  const void* cmax_out, const void* cmax_in,
                                                  int total_count, int dim, float ratio,
                                                  lsh_stream_t stream);
int lsh_launch_ls_quant_dropout_act_bias_gelu_f32(int8_t* qout, uint8_t* cmask_out,
                                                  uint8_t* cmask_in, uint8_t* dropout_mask,
                                                  const int8_t* qinput, const void* bias,
                                                  const void* cmax_out, const void* cmax_in,
                                                  int total_count, int dim, float ratio,
                                                  lsh_stream_t stream);
int lsh_launch_ls_quant_dropout_act_bias_relu_f16(int8_t* qout, uint8_t* cmask_out,
                                                  uint8_t* cmask_in, uint8_t* dropout_mask,
                                                  const int8_t* qinput, const void* bias,
                                                  const void* cmax_out, const void* cmax_in,
                                                  int total_count, int dim, float ratio,
                                                  lsh_stream_t stream);
int lsh_launch_ls_quant_dropout_act_bias_relu_f32(int8_t* qout, uint8_t* cmask_out,
                                                  uint8_t* cmask_in, uint8_t* dropout_mask,
                                                  const int8_t* qinput, const void* bias,
                                                  const void* cmax_out, const void* cmax_in,
                                                  int total_count, int dim, float ratio,
                                                  lsh_stream_t stream);
/* kernels.h:146-151 launch_ls_fakequant_dropout_act_bias<act> (dropout_kernels.cu:1078-1302) */
int lsh_launch_ls_fakequant_dropout_act_bias_gelu_f16(void* out, uint8_t* cmask_out,
                                                      uint8_t* cmask_in, uint8_t* dropout_mask,
                                                      const int8_t* qinput, const void* bias,
                                                      const void* cmax_out, const void* cmax_in,
                                                      int total_count, int dim, float ratio,
                                                      lsh_stream_t stream, int in_col32,
                                                      int symmetry);
int lsh_launch_ls_fakequant_dropout_act_bias_gelu_f32(void* out, uint8_t* cmask_out,
                                                      uint8_t* cmask_in, uint8_t* dropout_mask,
                                                      const int8_t* qinput, const void* bias,
                                                      const void* cmax_out, const void* cmax_in,
                                                      int total_count, int dim, float ratio,
                                                      lsh_stream_t stream, int in_col32,
                                                      int symmetry);
int lsh_launch_ls_fakequant_dropout_act_bias_relu_f16(void* out, uint8_t* cmask_out,
                                                      uint8_t* cmask_in, uint8_t* dropout_mask,
                                                      const int8_t* qinput, const void* bias,
                                                      const void* cmax_out, const void* cmax_in,
                                                      int total_count, int dim, float ratio,
                                                      lsh_stream_t stream, int in_col32,
                                                      int symmetry);
int lsh_launch_ls_fakequant_dropout_act_bias_relu_f32(void* out, uint8_t* cmask_out,
                                                      uint8_t* cmask_in, uint8_t* dropout_mask,
                                                      const int8_t* qinput, const void* bias,
                                                      const void* cmax_out, const void* cmax_in,
                                                      int total_count, int dim, float ratio,
                                                      lsh_stream_t stream, int in_col32,
                                                      int symmetry);
/* kernels.h:153-159 launch_ls_quant_dropout_res_bias (dropout_kernels.cu:1808-1967) */
int lsh_launch_ls_quant_dropout_res_bias_f16(void* out, uint8_t* mask, const int8_t* qvals,
                                             const void* cmax, const void* bias,
                                             const void* residual, int total_count, int dim,
                                             float ratio, lsh_stream_t stream, int in_col32);
int lsh_launch_ls_quant_dropout_res_bias_f32(void* out, uint8_t* mask, const int8_t* qvals,
                                             const void* cmax, const void* bias,
                                             const void* residual, int total_count, int dim,
                                             float ratio, lsh_stream_t stream, int in_col32);

/* ---- int8 GEMM with device-resident scale ----------------------------------------------------- */
/* cublaslt_igemm<int8_t, float> / cublasLtMM_withAlgo_i8IO of
 * kernels/cuda/cublas_wrappers.cpp:98-559 as FeedForward<T>::Forward calls them
 * (ops/includes/feed_forward.h:46-79): qout[bsz, out] = sat(alpha[0] * qin[bsz, in] x
 * qweight[out, in]^T), alpha in device memory; beta must point to 0 or be null. */
int lsh_feed_forward_i8(int bsz, int output_size, int input_size, const int8_t* qinput_ptr,
                        const int8_t* qweight_ptr, const float* alpha_ptr, const float* beta_ptr,
                        int8_t* qout_ptr, lsh_stream_t stream);
/* StridedBatchGemm<T>::Forward (ops/includes/strided_batch_gemm.h:45-57 over
 * cublas_strided_batched_gemm, kernels/cuda/cublas_wrappers.cpp): per batch element, in
 * column-major terms, output (m x n) = alpha * op(A) (m x k) * op(B) (k x n) + beta * output,
 * with strides m*k, n*k, m*n; op_a / op_b: 0 = N, 1 = T (the values of cublasOperation_t).
 * The layers configure it as (T, N; m = to_len, n = from_len, k = head_dim; alpha =
 * 1/sqrt(head_dim)) for the scores and (N, N; m = head_dim, n = from_len, k = to_len) for the
 * context (layers/transformer_encoder_layer.cpp:34-42, :121-141). */
int lsh_strided_batch_gemm_f16(int bsz, int m, int n, int k, float alpha, float beta, int op_a,
                               int op_b, const void* buffer_a, const void* buffer_b,
                               void* output, lsh_stream_t stream);
int lsh_strided_batch_gemm_f32(int bsz, int m, int n, int k, float alpha, float beta, int op_a,
                               int op_b, const void* buffer_a, const void* buffer_b,
                               void* output, lsh_stream_t stream);
/* Attention core of the layer in one kernel, fp16: replaces StridedBatchGemm (scores) +
 * launch_attn_softmax + Dropout::dropout + StridedBatchGemm (context) +
 * launch_transform4d_0213 of layers/transformer_encoder_layer.cpp:121-148.  No single
 * counterpart in the reference.  q, k, v: [batch, heads, seq_len, dim_per_head];
 * attn_mask [batch, seq_len] additive or null; ctx: [batch, seq_len, heads * dim_per_head]. */
int lsh_layer_attention_f16(const void* q, const void* k, const void* v, const void* attn_mask,
                            void* ctx, int batch_size, int seq_len, int heads, int dim_per_head,
                            int mask_future, lsh_stream_t stream);
/* The same with its own number of keys, as the decoder layer needs it
 * (layers/transformer_decoder_layer.cpp:173-189 a cached decoding step: from_len 1, to_len
 * step + 1; :333-357 cross attention: to_len = source length).  q: [batch, heads, from_len,
 * dim_per_head]; k, v: [batch, heads, to_len, dim_per_head]; attn_mask [batch, to_len] additive
 * or null; ctx: [batch, from_len, heads * dim_per_head].  mask_future needs from_len == to_len. */
int lsh_layer_cross_attention_f16(const void* q, const void* k, const void* v,
                                  const void* attn_mask, void* ctx, int batch_size, int from_len,
                                  int to_len, int heads, int dim_per_head, int mask_future,
                                  lsh_stream_t stream);

/* ---- layers (pybind/pybind_layer.cpp) ----------------------------------------------------------- */
/* Context::Instance().set_stream (ops/includes/context.h:14-43): the stream every layer
 * created afterwards launches on (null = the default stream). */
int ls_layer_set_stream(lsh_stream_t stream);
/* pybind_layer.cpp:28-50 create_transformer_encoder_layer<__half>: registers a
 * TransformerEncoderLayer (layers/includes/transformer_encoder_layer.h:20-33) under
 * layer_id.  activation_fn is "relu" or "gelu". */
int ls_create_transformer_encoder_layer_fp16(int layer_id, int max_batch_tokens, int max_seq_len,
                                             int hidden_dim, int num_heads, int intermediate_size,
                                             float attn_prob_dropout_ratio,
                                             float activation_dropout_ratio,
                                             float hidden_dropout_ratio, int is_pre_ln,
                                             const char* activation_fn, int mask_future_tokens);
/* pybind_layer.cpp:52-73 transformer_encoder_layer_fw<__half>: input fp16 [batch, seq_len,
 * hidden], input_mask fp16 [batch, seq_len] additive, output fp16 like input (caller
 * allocated).  training_mode must be 0; quant_mode must be 1 (the float path of the layer is
 * outside this library). */
int ls_transformer_encoder_layer_fw_fp16(int layer_id, const void* input, const void* input_mask,
                                         void* output, int batch_size, int seq_len,
                                         int training_mode, int prelayernorm, int quant_mode);
/* pybind_layer.cpp:110-132 create_transformer_decoder_layer<__half>: registers a
 * TransformerDecoderLayer (layers/includes/transformer_decoder_layer.h:19-32) under layer_id.
 * Create every decoder layer of a stack before binding the parameters of layer 0: its blob
 * holds the cross-attention k/v projection of all of them. */
int ls_create_transformer_decoder_layer_fp16(int layer_id, int max_batch_tokens, int max_seq_len,
                                             int hidden_dim, int num_heads, int intermediate_size,
                                             float attn_prob_dropout_ratio,
                                             float activation_dropout_ratio,
                                             float hidden_dropout_ratio, int is_pre_ln,
                                             const char* activation_fn);
/* pybind_layer.cpp:134-185 transformer_decoder_layer_fw<__half>.  step < 0: the whole target
 * sequence, dec_input fp16 [batch, trg_seq_len, hidden], cache null.  step >= 0: one decoding
 * step, trg_seq_len is the beam size, dec_input [batch * beam, 1, hidden] and cache points to
 * 5 device pointers: new k, new v [batch * beam * heads, step + 1, head_dim] (written),
 * previous k, v [.., step, head_dim] (read; may be null at step 0), and, for layer 0, the
 * cross-attention k/v of all layers [layers * 2, batch, heads, src_seq_len, head_dim] (written
 * at step 0).  enc_output fp16 [batch, src_seq_len, hidden] is read by layer 0 only;
 * enc_mask fp16 [batch, src_seq_len] additive or null.  The reference derives step and the
 * lengths from its tensor arguments; here they are explicit.  training_mode must be 0 and
 * quant_mode 1. */
int ls_transformer_decoder_layer_fw_fp16(int layer_id, const void* dec_input,
                                         const void* enc_output, const void* enc_mask,
                                         void* dec_output, int batch_size, int trg_seq_len,
                                         int src_seq_len, int step, void* const* cache,
                                         int training_mode, int prelayernorm, int quant_mode);
/* Number of fp16 elements the parameter blob of a registered layer holds ("TransformerEncoderLayer"
 * or "TransformerDecoderLayer"), written to *count; no counterpart in the reference, whose
 * Python side computes it. */
int ls_layer_param_count(const char* layer_name, int layer_id, long long* count);
/* pybind_layer.cpp assign_layer_weight_grad<__half>: binds the flat fp16 parameter blob of
 * layer "TransformerEncoderLayer" (transformer_encoder_layer.h:66-105: qkvw, qkvb, ow, ob, nw,
 * nb, inter_w, inter_b, out_w, out_b, ffn_nw, ffn_nb, 12 clip_max) or "TransformerDecoderLayer"
 * (transformer_decoder_layer.h:100-168: self attention qkvw, qkvb, ow, ob, nw, nb; cross
 * attention qw, qb, ow, ob, nw, nb; inter_w, inter_b, out_w, out_b, ffn_nw, ffn_nb; 24
 * clip_max; layer 0: kvw, kvb of all layers); the gradient blob is accepted and ignored. */
int ls_assign_layer_weight_grad_fp16(const void* weights, void* grads, const char* layer_name,
                                     int layer_id);
/* pybind_layer.cpp create_quant_linear_layer<__half> / quant_linear_layer_fw<__half>
 * (layers/quant_linear_layer.cpp:7-45): outputs[tokens, out] = dequantize(sat(alpha *
 * quantize(inputs) x quantize(weight)^T), clip_max[2]); clip_max: 3 fp16 device scalars. */
int ls_create_quant_linear_layer_fp16(int layer_id, int in_features, int out_features,
                                      int max_batch_tokens);
int ls_quant_linear_layer_fw_fp16(int layer_id, const void* inputs, const void* weight,
                                  const void* clip_max, void* outputs, int batch_size, int seq_len,
                                  int quant_mode);
/* Releases a layer and its buffers (the reference keeps them until the process ends). */
int ls_destroy_layer(const char* layer_name, int layer_id);

#ifdef __cplusplus
}
#endif
#endif /* LIGHTSEQ_OPS_H_ */
