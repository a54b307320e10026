/*
 * lightseq_hip.h -- C ABI of the MI355X (gfx950) int8 transformer-layer forward path.
 *
 * Every entry point replaces one launcher / helper of the reference
 * (bytedance/lightseq v3.0.1; paths below are relative to lightseq/inference/
 * unless noted).  Argument names, order and meaning follow the reference
 * launcher, with three systematic changes:
 *   - the template parameter T in {float, __half} becomes a _f32 / _f16 suffix and
 *     T-typed pointers become void*;
 *   - cudaStream_t becomes lsh_stream_t (a hipStream_t);
 *   - every function returns an int status (LSH_OK == 0) instead of void, and a
 *     description of the last failure on the calling thread is available from
 *     lsh_last_error().  Where the reference throws (bad sampling k, hidden % 8,
 *     batch > max_batch ...) the status is LSH_ERR_INVALID with the same message.
 * The cuBLASLt-specific COL32 layouts do not exist here: a call with an
 * in_col32 / out_col32 flag set returns LSH_ERR_UNSUPPORTED.
 *
 * All pointers are device pointers unless a parameter is documented as host.
 * Launchers are asynchronous on `stream`, allocate nothing and never synchronise.
 */
#ifndef LIGHTSEQ_HIP_H_
#define LIGHTSEQ_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* lsh_stream_t;

enum {
  LSH_OK = 0,
  LSH_ERR_INVALID = 1,     /* violated precondition (the reference throws or misbehaves) */
  LSH_ERR_UNSUPPORTED = 2, /* valid in the reference, not provided here (COL32 layouts ...) */
  LSH_ERR_HIP = 3,         /* a HIP runtime call failed */
  LSH_ERR_IO = 4           /* model file could not be read / parsed */
};

/* Message of the last non-OK status returned on this thread ("" if none). */
const char* lsh_last_error(void);
/* Library version string and the gfx architecture the kernels were built for. */
const char* lsh_version(void);

/* ---- quantise / dequantise --------------------------------------------------- */
/* kernels/transformerKernels_int8.h:11-14 */
int lsh_launch_quantize_tensor_f16(const void* input, int8_t* output, int batch_tokens,
                                   int hidden_size, float quant_scale, lsh_stream_t stream,
                                   int out_col32);
int lsh_launch_quantize_tensor_f32(const void* input, int8_t* output, int batch_tokens,
                                   int hidden_size, float quant_scale, lsh_stream_t stream,
                                   int out_col32);
/* kernels/transformerKernels_int8.h:16-19 */
int lsh_launch_dequantize_tensor_f16(const int32_t* input, void* output, int batch_tokens,
                                     int hidden_size, float dequant_scale, lsh_stream_t stream,
                                     int in_col32);
int lsh_launch_dequantize_tensor_f32(const int32_t* input, void* output, int batch_tokens,
                                     int hidden_size, float dequant_scale, lsh_stream_t stream,
                                     int in_col32);

/* ---- LayerNorm family ---------------------------------------------------------- */
/* kernels/transformerKernels_int8.h:21-26 */
int lsh_ker_norm_layer_resual_i8O_f16(int token_num, int hidden_size, lsh_stream_t stream,
                                      void* input, int8_t* output, const void* scale,
                                      const void* bias, const void* residual_bias,
                                      int max_thread_per_block, float quant_scale, int is_post_ln,
                                      int out_col32);
int lsh_ker_norm_layer_resual_i8O_f32(int token_num, int hidden_size, lsh_stream_t stream,
                                      void* input, int8_t* output, const void* scale,
                                      const void* bias, const void* residual_bias,
                                      int max_thread_per_block, float quant_scale, int is_post_ln,
                                      int out_col32);
/* kernels/transformerKernels_int8.h:47-53 */
int lsh_ker_residual_bias_ln_i32I_i8O_f16(const int32_t* input, const void* scale,
                                          const void* bias, const void* residual_bias,
                                          int8_t* output, void* residual, int batch_tokens,
                                          int hidden_size, float dequant_scale, float quant_scale,
                                          int max_thread_per_block, lsh_stream_t stream,
                                          int is_post_ln, int in_col32, int out_col32,
                                          const void* colsum);
int lsh_ker_residual_bias_ln_i32I_i8O_f32(const int32_t* input, const void* scale,
                                          const void* bias, const void* residual_bias,
                                          int8_t* output, void* residual, int batch_tokens,
                                          int hidden_size, float dequant_scale, float quant_scale,
                                          int max_thread_per_block, lsh_stream_t stream,
                                          int is_post_ln, int in_col32, int out_col32,
                                          const void* colsum);
/* kernels/transformerKernels_int8.h:55-61 */
int lsh_ker_residual_bias_ln_i8I_i8O_f16(const int8_t* input, const void* scale, const void* bias,
                                         const void* residual_bias, int8_t* output, void* residual,
                                         int batch_tokens, int hidden_size, float dequant_scale,
                                         float quant_scale, int max_thread_per_block,
                                         lsh_stream_t stream, int is_post_ln, int in_col32,
                                         int out_col32, const void* colsum);
int lsh_ker_residual_bias_ln_i8I_i8O_f32(const int8_t* input, const void* scale, const void* bias,
                                         const void* residual_bias, int8_t* output, void* residual,
                                         int batch_tokens, int hidden_size, float dequant_scale,
                                         float quant_scale, int max_thread_per_block,
                                         lsh_stream_t stream, int is_post_ln, int in_col32,
                                         int out_col32, const void* colsum);
/* kernels/transformerKernels_int8.h:63-68 (output may alias residual) */
int lsh_ker_residual_bias_ln_i32I_f16(const int32_t* input, const void* scale, const void* bias,
                                      const void* residual, void* output, int batch_tokens,
                                      int hidden_size, float dequant_scale,
                                      int max_thread_per_block, lsh_stream_t stream, int in_col32,
                                      const void* colsum);
int lsh_ker_residual_bias_ln_i32I_f32(const int32_t* input, const void* scale, const void* bias,
                                      const void* residual, void* output, int batch_tokens,
                                      int hidden_size, float dequant_scale,
                                      int max_thread_per_block, lsh_stream_t stream, int in_col32,
                                      const void* colsum);

/* ---- bias + activation + requant ------------------------------------------------ */
/* kernels/transformerKernels_int8.h:29-35 */
int lsh_ker_bias_gelu_i8I_i8O_f16(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, int in_col32,
                                  int out_col32);
int lsh_ker_bias_gelu_i8I_i8O_f32(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, int in_col32,
                                  int out_col32);
/* kernels/transformerKernels_int8.h:38-45 */
int lsh_ker_bias_relu_i8I_i8O_f16(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, float clip_max,
                                  int in_col32, int out_col32, int narrow_clip);
int lsh_ker_bias_relu_i8I_i8O_f32(int batch_token_num, lsh_stream_t stream, const int8_t* input,
                                  int8_t* output, const void* bias, int feature_dim,
                                  float dequant_scale, float quant_scale, float clip_max,
                                  int in_col32, int out_col32, int narrow_clip);

/* ---- head split / merge ----------------------------------------------------------- */
/* kernels/transformerKernels_int8.h:70-75 */
int lsh_ker_arrange_encself_qkv_i8I_f16(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                        const int8_t* ori_qkv, const void* qkv_bias, void* new_qkv,
                                        int max_batch_dim, int batch_seq_len, int dim_per_head,
                                        int head_num, int max_thread_per_block,
                                        float dequant_scale, int in_col32);
int lsh_ker_arrange_encself_qkv_i8I_f32(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                        const int8_t* ori_qkv, const void* qkv_bias, void* new_qkv,
                                        int max_batch_dim, int batch_seq_len, int dim_per_head,
                                        int head_num, int max_thread_per_block,
                                        float dequant_scale, int in_col32);
/* kernels/transformerKernels_int8.h:77-83 */
int lsh_ker_arrange_encself_qkv_i8I_i8O_f16(int batch_token_num, int hidden_size,
                                            lsh_stream_t stream, const int8_t* ori_qkv,
                                            const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                            int8_t* new_v, void* d_v, int batch_seq_len,
                                            int dim_per_head, int head_num,
                                            int max_thread_per_block, float dequant_scale,
                                            float quant_scale, int in_col32);
int lsh_ker_arrange_encself_qkv_i8I_i8O_f32(int batch_token_num, int hidden_size,
                                            lsh_stream_t stream, const int8_t* ori_qkv,
                                            const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                            int8_t* new_v, void* d_v, int batch_seq_len,
                                            int dim_per_head, int head_num,
                                            int max_thread_per_block, float dequant_scale,
                                            float quant_scale, int in_col32);
/* kernels/transformerKernels_int8.h:85-89 */
int lsh_ker_arrange_atten_output_i8O_f16(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                         const void* ori_q, int8_t* new_q, int beam_size,
                                         int dim_per_head, int head_num, int max_thread_per_block,
                                         float quant_scale, int out_col32);
int lsh_ker_arrange_atten_output_i8O_f32(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                         const void* ori_q, int8_t* new_q, int beam_size,
                                         int dim_per_head, int head_num, int max_thread_per_block,
                                         float quant_scale, int out_col32);

/* ---- encoder attention core --------------------------------------------------------- */
/* kernels/transformerKernels.h (ker_correlation_softmax_encself_launcher),
 * kernels/transformerKernels.cc.cu:1119-1172 */
int lsh_ker_correlation_softmax_encself_f16(int batch_size, int batch_seq_len, int head_num,
                                            lsh_stream_t stream, void* correlation,
                                            const int* src_padding_mask);
int lsh_ker_correlation_softmax_encself_f32(int batch_size, int batch_seq_len, int head_num,
                                            lsh_stream_t stream, void* correlation,
                                            const int* src_padding_mask);
/* Fused replacement of the sequence at model/quant_bert_encoder.cc.cu:321-347
 * (cublasGemmStridedBatchedEx K^T Q, ker_correlation_softmax_encself,
 * cublasGemmStridedBatchedEx V P, ker_arrange_atten_output_i8O).  q, k, v are
 * [batch, head_num, seq_len, dim_per_head] fp16.  ctx ([batch, head_num, seq_len,
 * dim_per_head] fp16) and ctx_q ([batch*seq_len, head_num*dim_per_head] int8,
 * quantised with quant_scale) are each optional (NULL), not both. */
int lsh_encself_attention_f16(const void* q, const void* k, const void* v,
                              const int* src_padding_mask, void* ctx, int8_t* ctx_q,
                              float quant_scale, int batch_size, int batch_seq_len, int head_num,
                              int dim_per_head, lsh_stream_t stream);
/* The same sequence preceded by ker_arrange_encself_qkv_i8I
 * (kernels/transformerKernels_int8.cc.cu:1119-1172; call site
 * model/quant_bert_encoder.cc.cu:313-319): qkv is the int8 output of the QKV product,
 * [batch*seq_len, 3*hidden], qkv_bias fp16 [3*hidden]; each element is dequantised to
 * half(half(code * dequant_scale) + bias) as it is read, so the fp16 q, k, v tensors
 * are never written. */
int lsh_encself_attention_i8qkv_f16(const int8_t* qkv, const void* qkv_bias, float dequant_scale,
                                    const int* src_padding_mask, void* ctx, int8_t* ctx_q,
                                    float quant_scale, int batch_size, int batch_seq_len,
                                    int head_num, int dim_per_head, lsh_stream_t stream);

/* The QKV projection and the attention above in one kernel, for heads of 64 dimensions,
 * sequences of at most 128 tokens and hidden % 128 == 0 (LSH_ERR_UNSUPPORTED otherwise):
 * x int8 [batch*seq_len, hidden], qkv_weight int8 [3*hidden, hidden]; requant_alpha is the
 * alpha of the int8-output GEMM (quant_bert_encoder.cc.cu:305-319), dequant_scale the one
 * of ker_arrange_encself_qkv_i8I.  Replaces quant_bert_encoder.cc.cu:305-347 in one launch;
 * the result is byte-identical to lsh_gemm_i8_i8o followed by
 * lsh_encself_attention_i8qkv_f16. */
int lsh_qkv_attention_i8_f16(const int8_t* x, const int8_t* qkv_weight, const void* qkv_bias,
                             const int* src_padding_mask, int8_t* ctx_q, float requant_alpha,
                             float dequant_scale, float quant_scale, int batch_size,
                             int batch_seq_len, int head_num, int dim_per_head,
                             lsh_stream_t stream);

/* The same launch with a plan made from the padding mask (no counterpart in the reference).
 * The context of a padded query is zero whatever its q is, and a padded key contributes exactly
 * nothing (kernels/transformerKernels.cc.cu:1119-1172), so a workgroup leaves out the 32-token
 * blocks of its sequence that hold nothing but padding -- in the product, in the conversion and
 * in the attention -- and the plan deals the (sequence, head) pairs out longest sequence first,
 * so that the compute units that hold two workgroups hold a long and a short one.  Bytes: those
 * of lsh_qkv_attention_i8_f16 on the rows of tokens that are not padding, zeros on the others
 * (there the unplanned launch leaves zeros too).  plan: batch_size * head_num ints of device
 * memory, written by lsh_qkv_attention_plan, valid for launches with that mask, batch_size,
 * batch_seq_len and head_num; batch_size <= 1024. */
int lsh_qkv_attention_plan(const int* src_padding_mask, int* plan, int batch_size,
                           int batch_seq_len, int head_num, lsh_stream_t stream);
/* whether the encoder models make and use a plan (default) -- an A/B switch; returns the
 * previous setting */
int lsh_qkv_attention_plan_in_models(int on);
int lsh_qkv_attention_planned_i8_f16(const int8_t* x, const int8_t* qkv_weight, const void* qkv_bias,
                                     const int* src_padding_mask, const int* plan, int8_t* ctx_q,
                                     float requant_alpha, float dequant_scale, float quant_scale,
                                     int batch_size, int batch_seq_len, int head_num,
                                     int dim_per_head, lsh_stream_t stream);

/* ---- embedding ------------------------------------------------------------------------ */
/* kernels/embKernels_int8.h:7-13 */
int lsh_launch_enc_emb_i8I_f16(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               void* output, int* pad_mask, int pad_id, int batch_size,
                               int seq_len, int hidden_dim, lsh_stream_t stream,
                               const void* lang_emb, const int* lang_id, int multilg_type,
                               float dequant_scale, int scaled);
int lsh_launch_enc_emb_i8I_f32(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               void* output, int* pad_mask, int pad_id, int batch_size,
                               int seq_len, int hidden_dim, lsh_stream_t stream,
                               const void* lang_emb, const int* lang_id, int multilg_type,
                               float dequant_scale, int scaled);
/* kernels/transformerKernels.h:15-17 */
int lsh_launch_scaled_colsum_f16(const void* inp, void* out, int rows, int cols, float scale,
                                 lsh_stream_t stream);
int lsh_launch_scaled_colsum_f32(const void* inp, void* out, int rows, int cols, float scale,
                                 lsh_stream_t stream);

/* ---- int8 GEMM (replaces cuBLASLt + the tuned-algorithm map) ---------------------------- */
/* C[m,n] = A[m,k] * W[n,k]^T with A (activations) and W (weights) K-contiguous.
 * model/cublas_helper.h:21-34 cublasLtMM_withAlgo (int32 out) and
 * model/cublas_helper.h:50-58 cublaslt_gemm<int32_t,int32_t>. */
int lsh_gemm_i8_i32o(const int8_t* A, const int8_t* W, int32_t* C, int m, int n, int k,
                     lsh_stream_t stream);
/* Selects, for the calling thread's later layer-norm launches (the lsh_ker_norm_layer_* and
 * lsh_ker_residual_bias_ln_* entry points, hidden <= 1024, 16-byte aligned operands), the
 * kernel that gives a workgroup to each row: its small code starts faster on launches of a
 * few rows (decode steps).  It adds a row's elements in another order than the default
 * kernel, so keep one setting for all launches whose results are compared with each other.
 * Returns the previous setting (0 / 1).  No counterpart in the reference. */
int lsh_layer_norm_row_kernel(int on);
/* Process-wide switch (default on; returns the previous setting, 0 / 1): products with
 * thousands of rows and columns run one 256 x 192 / 256 x 256 / 256 x 128 output tile per
 * workgroup on 8 wavefronts; off sends them to the persistent 128 x 64 / 128 x 128 kernels
 * instead.  Results are identical either way (integer sums); the switch exists to measure
 * one against the other.  No counterpart in the reference (its cuBLASLt algorithm table
 * plays this part: model/cublas_algo_map.cc). */
int lsh_gemm_i8_tile_kernel(int on);
/* Process-wide switch (default on; returns the previous setting, 0 / 1): products of at most
 * 64 rows (decode steps) whose K range per workgroup is a multiple of 256 run on 16 x 16 x 64
 * matrix instructions, where a load instruction of a wavefront reads whole 64-byte segments of
 * 16 weight rows; off sends them to the 32 x 32 x 32 kernel that serves the other K.  Results
 * are identical either way (integer sums).  No counterpart in the reference. */
int lsh_gemm_i8_decode_kernel_16x16(int on);
/* Process-wide switch (default on; returns the previous setting, 0 / 1): with at least 1024
 * rows and a feature dimension that is a multiple of 64, lsh_ker_bias_gelu_i8I_i8O_* tabulates
 * the 256 codes of each column per workgroup in LDS and looks the elements up instead of
 * evaluating the GELU per element.  The table comes from the same routine, so the results are
 * the same bytes; the switch exists to measure and to test one against the other.  No
 * counterpart in the reference. */
int lsh_bias_act_lut_kernel(int on);
/* The attention out-projection and the LayerNorm after it as one kernel: what
 * lsh_gemm_i8_i8o(A, W, alpha) followed by lsh_ker_residual_bias_ln_i8I_i8O_f16 leaves in
 * `output` (int8 [batch_tokens, hidden_size]) and `residual`, byte for byte (the product is
 * requantised to its int8 code before the dequant + residual, as
 * inference/model/quant_bert_encoder.cc.cu:361-396 does), without the int8 product ever
 * reaching memory.  hidden_size == k in {512, 768, 1024}; w_tiled is W [hidden_size, k]
 * re-ordered once by lsh_tile_weight_16x64 (blocks of 16 rows x 64 bytes in MFMA lane order).
 * No counterpart in the reference. */
int lsh_tile_weight_16x64(const int8_t* w, int8_t* tiled, int n, int k, lsh_stream_t stream);
int lsh_gemm_i8_residual_ln_i8O_f16(const int8_t* A, const int8_t* w_tiled, float alpha,
                                    const void* scale, const void* bias, const void* residual_bias,
                                    int8_t* output, void* residual, int batch_tokens,
                                    int hidden_size, int k, float dequant_scale, float quant_scale,
                                    lsh_stream_t stream, int is_post_ln);
/* The feed-forward half of an encoder layer as one launch, no counterpart in the reference
 * (it replaces three launches of model/quant_bert_encoder.cc.cu:414-520 and leaves their bytes):
 *   act = lut1[ requant(x W1^T, alpha1) ]       int8 [m, inner]   (lsh_gemm_i8_lut_i8o)
 *   acc = act W2^T                              int32 [m, hidden] (lsh_gemm_i8_i32o)
 *   final_ln == 0: lsh_ker_residual_bias_ln_i32I_i8O_f16(acc, scale, bias, residual_bias, out_q,
 *                  residual, ..., is_post_ln, colsum);
 *   final_ln != 0: lsh_ker_residual_bias_ln_i32I_f16(acc, scale, bias, residual, out_t, ...,
 *                  colsum) (out_t may alias residual; residual_bias and out_q unused).
 * The token rows are dealt to the GPU's 8 XCDs; the 32 workgroups of an XCD wait for one another
 * between the three phases through the L2 they share.  Needs a GPU of 256 compute units that
 * each hold a workgroup of the kernel (otherwise LSH_ERR_UNSUPPORTED), hidden and inner
 * multiples of 128, hidden <= 1024, m >= 8.
 * sync: lsh_ffn_segment_sync_words() uint32 words of device memory that the caller zeroes
 * once; *launches: the caller's count of launches that used `sync` (starts at 0, advanced by
 * the call).  Every wait inside the kernel is bounded by spin_limit polls (about a microsecond
 * each): if the workgroups cannot all become resident -- another kernel of this kind running
 * at the same time -- the kernel gives up, sets sync[words - 1] (bit 0: a wait gave up, bit 1:
 * two workgroups found themselves in the same place of an XCD) and ends; the outputs are then
 * undefined, and `sync` and *launches must be zeroed before the next call.  Calls that overlap
 * on one GPU must not share `sync`. */
/* What the encoder models do where the shape is covered: the three launches (default: the
 * segment kernel measured no faster, 38.9 us against 39.4 us per BERT-base layer at batch 32 x
 * 128) or the segment kernel; returns the previous setting.  A model that saw the kernel give up leaves it
 * for good.  At most one model of a process runs it at a time (a second one that starts an
 * Infer() meanwhile takes the three launches). */
int lsh_ffn_segment_in_models(int on);
/* Measurement aid: while `dev` (device memory, 256 x 8 uint64) is set, every launch of the
 * segment kernel records per workgroup the 100 MHz clock at: 0 its start, 1 FFN1 done, 2 past
 * the first barrier, 3 FFN2 done, 4 past the second barrier, 5 layer norm done.  NULL: off. */
int lsh_ffn_segment_stamps(uint64_t* dev);
size_t lsh_ffn_segment_sync_words(void);
int lsh_ffn_segment_supported(int m, int hidden, int inner);
int lsh_ffn_segment_i8_f16(const int8_t* x, const int8_t* w1, const int8_t* lut1, float alpha1,
                           int8_t* act, const int8_t* w2, int32_t* acc, void* residual, void* out_t,
                           int8_t* out_q, const void* scale, const void* bias,
                           const void* residual_bias, const void* colsum, int m, int hidden,
                           int inner, float dequant_scale, float quant_scale, int is_post_ln,
                           int final_ln, uint32_t* sync, uint32_t* launches, int spin_limit,
                           lsh_stream_t stream);
/* Measurement aid, no counterpart in the reference: one launch of `workgroups` x 4 wavefronts
 * that issue nothing but independent int8 MFMAs (v_mfma_i32_32x32x32_i8) on register-resident
 * operands, `iters` x 8 each.  out: workgroups * 256 ints (checksums, so that nothing is
 * optimised away); *ops receives the integer operations of the launch.  Timed by the caller:
 * ops / time is what the matrix units sustain at the clock the part holds under that load. */
int lsh_mfma_i8_peak_probe(int* out, int workgroups, int iters, double* ops, lsh_stream_t stream);
/* Decode-step QKV product with ker_arrange_decself_qkv_i8I_i8O
 * (kernels/transformerKernels_int8.cc.cu:1432-1513; call sites model/quant_decoder.cc.cu:660-674,
 * model/quant_gpt_encoder.cc.cu:640-653) as its epilogue: A [step_token_num, k] x W [3*hidden, k]
 * -> int8 code (alpha) -> code * dequant_scale + bias -> int8 (quant_scale); q codes to new_q
 * [step_token_num, hidden], k and v codes to slot step_id of the caches [step_token_num,
 * head_num, max_step, hidden/head_num].  Same bits as lsh_gemm_i8_i8o followed by
 * lsh_ker_arrange_decself_qkv_i8I_i8O_f16.  No counterpart in the reference. */
int lsh_gemm_i8_decself_qkv_i8o_f16(const int8_t* A, const int8_t* W, const void* qkv_bias,
                                    int8_t* new_q, int8_t* new_k, int8_t* new_v,
                                    int step_token_num, int hidden, int k, int head_num,
                                    int max_step, int step_id, float alpha, float dequant_scale,
                                    float quant_scale, lsh_stream_t stream);
/* lsh_gemm_i8_decself_qkv_i8o_f16 followed by lsh_decself_attention_i8 (step_num = step_id + 1)
 * as one launch, for heads of 64 dimensions, hidden % 128 == 0, hidden <= 1024 and max_step <=
 * 4096 (LSH_ERR_UNSUPPORTED otherwise): x int8 [rows, hidden] x qkv_weight [3*hidden, hidden]
 * -> q codes to new_q [rows, hidden], k and v codes to slot step_id of the caches [rows,
 * head_num, max_step, 64] (the same bytes as the stand-alone product), then the attention of
 * every (row, head) over slots 0..step_id -> int8 context codes ctx [rows, hidden] (the same
 * bytes as the stand-alone attention for caches of more than 128 and at most 256 steps; with
 * other lengths the value sums run in another tree and a code can differ by one next to a
 * rounding boundary).  alpha, dequant_scale, cache_quant_scale: the scales of the product;
 * attn_scale, cache_dequant_scale, ctx_quant_scale: those of the attention.  ctx must not alias
 * x.  Replaces the launches of model/quant_decoder.cc.cu:660-700 and
 * model/quant_gpt_encoder.cc.cu:640-680.  No counterpart in the reference. */
int lsh_decself_qkv_attention_i8_f16(const int8_t* x, const int8_t* qkv_weight,
                                     const void* qkv_bias, int8_t* new_q, int8_t* k_cache,
                                     int8_t* v_cache, int8_t* ctx, int rows, int hidden,
                                     int head_num, int max_step, int step_id, float alpha,
                                     float dequant_scale, float cache_quant_scale,
                                     float attn_scale, float cache_dequant_scale,
                                     float ctx_quant_scale, lsh_stream_t stream);
/* Process-wide switch (default off; returns the previous setting, 0 / 1): QuantTransformer and
 * QuantGpt run the decode-step self attention through lsh_decself_qkv_attention_i8_f16 where it
 * is supported, or through the two launches it replaces.  Off by default: measured on whole
 * generation runs the single launch is no faster than the pair (the projection of a head is
 * too little work to hide its weight stream).  No counterpart in the reference. */
int lsh_decself_qkv_attention_in_models(int on);
/* lsh_launch_dec_emb_i8I_vocab_major_f16 followed by lsh_ker_norm_layer_resual_i8O_f16 with the
 * row kernel selected (lsh_layer_norm_row_kernel(1)) as one launch, for the first layer of a
 * decode step (model/quant_decoder.cc.cu:570-580 + :620-633): tokens [rows, max_step] (column
 * `step` is read), token_emb int8 [vocab, hidden], pos_emb fp16 [max_step, hidden]; residual
 * [rows, hidden] receives what the layer norm leaves there (embedding, or the normalised row
 * when is_post_ln, + residual_bias), out_q the int8 codes.  The same bytes as the pair.
 * hidden % 4 == 0, hidden <= 1024, 16-byte aligned operands (LSH_ERR_UNSUPPORTED otherwise).
 * No counterpart in the reference. */
int lsh_dec_emb_norm_layer_i8O_f16(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                                   void* residual, int8_t* out_q, const void* scale,
                                   const void* bias, const void* residual_bias, int rows,
                                   int hidden, int vocab_size, int step, int max_step,
                                   float dequant_scale, int scaled, float quant_scale,
                                   int is_post_ln, lsh_stream_t stream);
/* lsh_launch_gpt_embedding_i8I_f16 for one position per sequence (batch_seq_len 1, pos_offset
 * `pos`) followed by lsh_ker_norm_layer_resual_i8O_f16 with the row kernel selected, as one
 * launch: the first layer of a cached GPT generation step (model/quant_gpt_encoder.cc.cu:363-377
 * + :215-225).  token_id [batch] (a padding token embeds to zeros and is not counted),
 * real_seq_len [batch] += 1 per counted token, zero_flag (may be NULL) cleared; residual
 * [batch, hidden] and out_q as lsh_dec_emb_norm_layer_i8O_f16.  The same bytes as the pair.
 * hidden % 4 == 0, hidden <= 1024, 16-byte aligned operands (LSH_ERR_UNSUPPORTED otherwise).
 * No counterpart in the reference. */
int lsh_gpt_emb_step_norm_layer_i8O_f16(const int8_t* token_emb, const void* pos_emb,
                                        const int* token_id, void* residual, int8_t* out_q,
                                        const void* scale, const void* bias,
                                        const void* residual_bias, int* real_seq_len,
                                        int* zero_flag, int batch_size, int hidden, int vocab_size,
                                        int padding_id, int pos, int max_step, float dequant_scale,
                                        float quant_scale, int is_post_ln, lsh_stream_t stream);
/* lsh_gemm_i8_encdec_q_f16 followed by lsh_encdec_attention_f16 (int8 context only) as one
 * launch (model/quant_decoder.cc.cu:745-800): x int8 [batch * beam, hidden], q_weight
 * [hidden, hidden], k / v fp16 [batch, head, batch_seq_len, 64], ctx_q int8 [batch * beam,
 * hidden] (must not overlap x).  The same bytes as the pair; the fp16 query is not stored.
 * Heads of 64, hidden <= 1024, at most 4 beams, batch_seq_len <= 128, 16-byte aligned operands
 * (LSH_ERR_UNSUPPORTED otherwise).  No counterpart in the reference. */
int lsh_encdec_q_attention_f16(const int8_t* x, const int8_t* q_weight, const void* q_bias,
                               const void* k, const void* v, const int* pad_mask, int8_t* ctx_q,
                               float quant_scale, int batch_size, int beam_size, int head_num,
                               int batch_seq_len, int hidden, float alpha, float dequant_scale,
                               lsh_stream_t stream);
/* Decode-step cross-attention query product with ker_arrange_encdec_q_i8I
 * (kernels/transformerKernels_int8.cc.cu:1596-1645; call site model/quant_decoder.cc.cu:745-760)
 * as its epilogue: A [step_token_num, k] x W [hidden, k] -> int8 code (alpha) ->
 * half(code * dequant_scale) + bias -> fp16 new_q [step_token_num / beam_size, head_num,
 * beam_size, hidden / head_num].  Same bits as lsh_gemm_i8_i8o followed by
 * lsh_ker_arrange_encdec_q_i8I_f16.  No counterpart in the reference. */
int lsh_gemm_i8_encdec_q_f16(const int8_t* A, const int8_t* W, const void* q_bias, void* new_q,
                             int step_token_num, int hidden, int k, int beam_size, int head_num,
                             float alpha, float dequant_scale, lsh_stream_t stream);
/* The bias + activation + requantisation epilogue as a table: after the requantisation an
 * element is one of 255 codes, so what follows depends only on (column, code).
 * lsh_build_act_lut fills lut [n, 256] (entry [col][code + 128]) with what
 * lsh_gemm_i8_bias_{gelu,relu}_i8o_f16 computes for that code (act: 0 GELU, 1 ReLU, 2 ReLU
 * with the narrow unsigned clip); lsh_gemm_i8_lut_i8o is the product with that table as its
 * epilogue, bit-identical to the arithmetic form and much cheaper per element.  Build the
 * table once per weight matrix.  No counterpart in the reference. */
int lsh_build_act_lut(int8_t* lut, const void* bias_f16, int n, float dequant_scale,
                      float quant_scale, float clip_max, int act, lsh_stream_t stream);
int lsh_gemm_i8_lut_i8o(const int8_t* A, const int8_t* W, int8_t* C, const int8_t* lut, int m,
                        int n, int k, float alpha, lsh_stream_t stream);
/* The int32 product with K split into `ksplit` equal ranges computed by different workgroups
 * (for shapes whose tile count would leave compute units idle, e.g. the second FFN product):
 * range p writes the plane C + p * m * n, so C needs ksplit * m * n elements; the planes are
 * summed by lsh_ker_residual_bias_ln_planes_i32I_i8O_f16 (integer sums: exact).  *used
 * receives the split actually applied (1 when k does not divide into whole 128-byte steps);
 * lsh_gemm_i8_preferred_ksplit returns the split the library would choose.  No counterpart
 * in the reference. */
int lsh_gemm_i8_i32o_splitk(const int8_t* A, const int8_t* W, int32_t* C, int m, int n, int k,
                            int ksplit, int* used, lsh_stream_t stream);
int lsh_gemm_i8_preferred_ksplit(int m, int n, int k);
/* lsh_ker_residual_bias_ln_i32I_i8O_f16 reading `nparts` accumulator planes `part_stride`
 * elements apart.  hidden_size % 8 == 0.  No counterpart in the reference. */
int lsh_ker_residual_bias_ln_planes_i32I_i8O_f16(const int32_t* input, int nparts,
                                                 int64_t part_stride, const void* scale,
                                                 const void* bias, const void* residual_bias,
                                                 int8_t* output, void* residual, int batch_tokens,
                                                 int hidden_size, float dequant_scale,
                                                 float quant_scale, lsh_stream_t stream,
                                                 int is_post_ln, const void* colsum);
/* int8 out: C = clamp(floor(float(acc) * alpha + 0.5), -127, 127).
 * model/cublas_helper.h:36-48 cublasLtMM_withAlgo_i8IO and
 * model/cublas_helper.h:50-58 cublaslt_gemm<int8_t,float>. */
int lsh_gemm_i8_i8o(const int8_t* A, const int8_t* W, int8_t* C, int m, int n, int k, float alpha,
                    lsh_stream_t stream);
/* Fused GEMM epilogues (fp16 storage).  No single counterpart in the reference: each is
 * the int8-output GEMM above followed, in the same kernel, by the launcher named below,
 * and produces exactly the bytes that pair produces (the intermediate int8 code is
 * formed in registers and never written to HBM).
 *  - lsh_gemm_i8_bias_gelu_i8o_f16 / lsh_gemm_i8_bias_relu_i8o_f16: FFN1 GEMM
 *    (model/quant_bert_encoder.cc.cu:415-431) + ker_bias_gelu_i8I_i8O_launcher /
 *    ker_bias_relu_i8I_i8O_launcher (:433-447); alpha as for lsh_gemm_i8_i8o, the
 *    remaining arguments as for the launcher.
 *  - lsh_gemm_i8_qkv_arrange_f16: QKV GEMM (:296-311) +
 *    ker_arrange_encself_qkv_i8I_launcher (:314-318); writes q, k, v as fp16
 *    [batch, head_num, seq_len, dim_per_head] at new_qkv + {0,1,2} * max_batch_dim.
 *    Needs dim_per_head % 16 == 0. */
int lsh_gemm_i8_bias_gelu_i8o_f16(const int8_t* A, const int8_t* W, int8_t* C, const void* bias,
                                  int m, int n, int k, float alpha, float dequant_scale,
                                  float quant_scale, lsh_stream_t stream);
int lsh_gemm_i8_bias_relu_i8o_f16(const int8_t* A, const int8_t* W, int8_t* C, const void* bias,
                                  int m, int n, int k, float alpha, float dequant_scale,
                                  float quant_scale, float clip_max, int narrow_clip,
                                  lsh_stream_t stream);
int lsh_gemm_i8_qkv_arrange_f16(const int8_t* A, const int8_t* W, void* new_qkv,
                                const void* qkv_bias, int max_batch_dim, int batch_token_num,
                                int hidden_size, int k, int batch_seq_len, int head_num,
                                float alpha, float dequant_scale, lsh_stream_t stream);
/* model/cublas_helper.h:60 quantize_weight: `origin_weight` is a HOST pointer to a
 * row-major [rows, cols] T matrix; it is uploaded, quantised with quant_scale and
 * stored at device pointer quantized_weight as [rows, cols] (layout 0, kRowMajor)
 * or transposed [cols, rows] (layout 1, kColMajor: the K-contiguous form the GEMMs
 * take).  Layout 2 (kColMajor32) is unsupported.  Synchronises `stream`. */
int lsh_quantize_weight_f16(const void* origin_weight, int8_t* quantized_weight, int rows,
                            int cols, float quant_scale, lsh_stream_t stream, int layout);
int lsh_quantize_weight_f32(const void* origin_weight, int8_t* quantized_weight, int rows,
                            int cols, float quant_scale, lsh_stream_t stream, int layout);

/* ======================================================================== */
/* decoder step                                                               */
/* ======================================================================== */

/* kernels/embKernels_int8.h launch_dec_emb_i8I (embKernels_int8.cc.cu:181-200).
 * tokens [batch*beam, max_step]; token_emb [hidden_dim, vocab_size] int8 codes;
 * output [batch*beam, hidden_dim] T.  multilg_type != 0 -> LSH_ERR_UNSUPPORTED
 * ("multilingle not supported", as the reference throws); step >= max_step ->
 * LSH_ERR_INVALID ("violate step < max_step").  The _vocab_major variants take the
 * table as [vocab_size, hidden_dim] -- the layout of the logits GEMM weight -- so one
 * copy of the shared embedding serves both uses and a row lookup is contiguous. */
int lsh_launch_dec_emb_i8I_f16(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               const void* lang_emb, const int* lang_id, void* output,
                               int batch_size, int beam_size, int hidden_dim, int vocab_size,
                               int step, int max_step, int multilg_type, lsh_stream_t stream,
                               float dequant_scale, int scaled);
int lsh_launch_dec_emb_i8I_f32(const int8_t* token_emb, const void* pos_emb, const int* tokens,
                               const void* lang_emb, const int* lang_id, void* output,
                               int batch_size, int beam_size, int hidden_dim, int vocab_size,
                               int step, int max_step, int multilg_type, lsh_stream_t stream,
                               float dequant_scale, int scaled);
int lsh_launch_dec_emb_i8I_vocab_major_f16(const int8_t* token_emb, const void* pos_emb,
                                           const int* tokens, const void* lang_emb,
                                           const int* lang_id, void* output, int batch_size,
                                           int beam_size, int hidden_dim, int vocab_size, int step,
                                           int max_step, int multilg_type, lsh_stream_t stream,
                                           float dequant_scale, int scaled);
int lsh_launch_dec_emb_i8I_vocab_major_f32(const int8_t* token_emb, const void* pos_emb,
                                           const int* tokens, const void* lang_emb,
                                           const int* lang_id, void* output, int batch_size,
                                           int beam_size, int hidden_dim, int vocab_size, int step,
                                           int max_step, int multilg_type, lsh_stream_t stream,
                                           float dequant_scale, int scaled);

/* kernels/transformerKernels_int8.h ker_arrange_decself_qkv_i8I_i8O_launcher
 * (transformerKernels_int8.cc.cu:1475-1486).  ori_qkv [step_token_num, 3*hidden] int8;
 * new_q [step_token_num, hidden]; new_k / new_v: slot step_id of the caches
 * [step_token_num, head_num, max_step, dim_per_head] int8. */
int lsh_ker_arrange_decself_qkv_i8I_i8O_f16(int step_token_num, int hidden_size,
                                            lsh_stream_t stream, const int8_t* ori_qkv,
                                            const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                            int8_t* new_v, int head_num, int dim_per_head,
                                            int max_step, int step_id, int max_thread_per_block,
                                            float dequant_scale, float quant_scale, int in_col32);
int lsh_ker_arrange_decself_qkv_i8I_i8O_f32(int step_token_num, int hidden_size,
                                            lsh_stream_t stream, const int8_t* ori_qkv,
                                            const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                            int8_t* new_v, int head_num, int dim_per_head,
                                            int max_step, int step_id, int max_thread_per_block,
                                            float dequant_scale, float quant_scale, int in_col32);

/* The strided-batched int8 GEMM of model/quant_decoder.cc.cu:676-683:
 * scores[bh, j] = sum_d q[bh, d] * k_cache[bh, j, d] for j < step_num, int32, row
 * stride max_step.  q [batch_head_num, dim_per_head], k_cache [batch_head_num,
 * max_step, dim_per_head]. */
int lsh_decself_scores_i8_i32o(const int8_t* k_cache, const int8_t* q, int32_t* scores,
                               int batch_head_num, int step_num, int max_step, int dim_per_head,
                               lsh_stream_t stream);
/* kernels/transformerKernels_int8.h ker_fuse_softmax_new_value_i32I_i8O_launcher
 * (transformerKernels_int8.cc.cu:1579-1594).  The value sum runs in ascending step
 * order (the reference accumulates with float atomics in no fixed order). */
int lsh_ker_fuse_softmax_new_value_i32I_i8O(const int32_t* correlation, const int8_t* v,
                                            int8_t* new_v, int batch_head_num, int step_num,
                                            int max_step, int head_num, int dim_per_head,
                                            float attn_scale, float dequant_scale,
                                            float quant_scale, int out_col32, lsh_stream_t stream);
/* The two calls above in one kernel (the int32 scores never reach HBM); produces the
 * bytes the pair produces.  No single counterpart in the reference. */
int lsh_decself_attention_i8(const int8_t* q, const int8_t* k_cache, const int8_t* v_cache,
                             int8_t* new_v, int batch_head_num, int step_num, int max_step,
                             int head_num, int dim_per_head, float attn_scale,
                             float dequant_scale, float quant_scale, lsh_stream_t stream);

/* kernels/transformerKernels_int8.h ker_arrange_encdec_q_i8I_launcher
 * (transformerKernels_int8.cc.cu:1653-1676).  new_q [batch, head_num, beam_size,
 * dim_per_head] T. */
int lsh_ker_arrange_encdec_q_i8I_f16(int step_token_num, int hidden_size, lsh_stream_t stream,
                                     const int8_t* ori_q, const void* q_bias, void* new_q,
                                     int beam_size, int dim_per_head, int head_num,
                                     int max_thread_per_block, float dequant_scale, int in_col32);
int lsh_ker_arrange_encdec_q_i8I_f32(int step_token_num, int hidden_size, lsh_stream_t stream,
                                     const int8_t* ori_q, const void* q_bias, void* new_q,
                                     int beam_size, int dim_per_head, int head_num,
                                     int max_thread_per_block, float dequant_scale, int in_col32);
/* kernels/transformerKernels.h ker_arrange_encdec_kv_launcher
 * (transformerKernels.cc.cu:985-1007).  ori_kv [batch_token_num, dec_layer_num, 2,
 * hidden] T; layer l of new_k / new_v starts l*offset_per_layer elements in and is
 * [batch, head_num, batch_seq_len, dim_per_head]. */
int lsh_ker_arrange_encdec_kv_f16(int batch_token_num, int dec_layer_num, int hidden_size,
                                  lsh_stream_t stream, const void* ori_kv, const void* kv_bias,
                                  void* new_k, void* new_v, int64_t offset_per_layer,
                                  int batch_seq_len, int dim_per_head, int head_num,
                                  int max_thread_per_block);
int lsh_ker_arrange_encdec_kv_f32(int batch_token_num, int dec_layer_num, int hidden_size,
                                  lsh_stream_t stream, const void* ori_kv, const void* kv_bias,
                                  void* new_k, void* new_v, int64_t offset_per_layer,
                                  int batch_seq_len, int dim_per_head, int head_num,
                                  int max_thread_per_block);
/* kernels/transformerKernels.h ker_correlation_softmax_encdec_launcher
 * (transformerKernels.cc.cu:1264-1276).  correlation [batch_size, head_num_per_seq,
 * batch_seq_len] T, in place; head_num_per_seq = head_num * beam_size. */
int lsh_ker_correlation_softmax_encdec_f16(int batch_size, int head_num_per_seq,
                                           int batch_seq_len, lsh_stream_t stream,
                                           void* correlation, const int* src_padding_mask);
int lsh_ker_correlation_softmax_encdec_f32(int batch_size, int head_num_per_seq,
                                           int batch_seq_len, lsh_stream_t stream,
                                           void* correlation, const int* src_padding_mask);
/* Fused encoder-decoder attention of one decoder layer (fp16): the two strided-batched
 * GEMMs, the softmax above and ker_arrange_atten_output_i8O of
 * model/quant_decoder.cc.cu:765-800 in one kernel, with the reference's fp16 rounding
 * points.  q [batch, head, beam, d]; k, v [batch, head, batch_seq_len, d]; ctx (same
 * layout as q) and ctx_q ([batch*beam, head*d] int8) are each optional. */
int lsh_encdec_attention_f16(const void* q, const void* k, const void* v, const int* pad_mask,
                             void* ctx, int8_t* ctx_q, float quant_scale, int batch_size,
                             int beam_size, int head_num, int batch_seq_len, int dim_per_head,
                             lsh_stream_t stream);
/* The cublasGemmEx of model/quant_decoder.cc.cu:497-501 in K-contiguous form:
 * C[m,n] = A[m,k] * W[n,k]^T, fp16 with fp32 accumulation.  k % 16 == 0. */
int lsh_gemm_f16_nt(const void* A, const void* W, void* C, int m, int n, int k,
                    lsh_stream_t stream);

/* ======================================================================== */
/* beam search                                                                */
/* ======================================================================== */

/* kernels/transformerKernels.h:137-140 length_norm (host). */
float lsh_length_norm(int length, float alpha);

/* kernels/transformerKernels_int8.h select_beam_rough_topk_i8I_launcher
 * (transformerKernels_int8.cc.cu:1846-1890).  Same buffers and candidate set as the
 * reference; candidates are written row by row in ascending vocabulary order (the
 * reference's order depends on atomics).  num_beam_can[0] = total,
 * num_beam_can[1 + row] = candidates of that row (not yet scanned).
 * max_thread_per_block defines the rough top-k threshold exactly as the reference's
 * block size does and must be a power of two in [32, 1024].  diverse_lambda != 0 ->
 * LSH_ERR_UNSUPPORTED. */
int lsh_select_beam_rough_topk_i8I_f16(const int8_t* logits, const void* logit_bias,
                                       const float* seq_probs, const float* seq_score,
                                       const int* alive_seq, float dequant_scale, int* can_idx,
                                       float* can_score, int* num_beam_can, int vocab_size,
                                       int max_step, float length_norm, int cur_step,
                                       int step_token_num, int max_thread_per_block,
                                       lsh_stream_t stream, int beam_size, float diverse_lambda,
                                       int end_id, int in_col32);
int lsh_select_beam_rough_topk_i8I_f32(const int8_t* logits, const void* logit_bias,
                                       const float* seq_probs, const float* seq_score,
                                       const int* alive_seq, float dequant_scale, int* can_idx,
                                       float* can_score, int* num_beam_can, int vocab_size,
                                       int max_step, float length_norm, int cur_step,
                                       int step_token_num, int max_thread_per_block,
                                       lsh_stream_t stream, int beam_size, float diverse_lambda,
                                       int end_id, int in_col32);
/* kernels/transformerKernels.h ker_refresh_result (transformerKernels.cc.cu:1398-1463;
 * launched at model/quant_decoder.cc.cu:1022-1027 with grid (batch_size, beam_size) and
 * max_step threads, given here as arguments).  Consumes candidates sorted by score,
 * descending, and the exclusively scanned per-row counts. */
int lsh_ker_refresh_result(const int* can_idx, const float* can_score,
                           const int* num_can_per_beam, const int* old_alive_seq,
                           int* new_alive_seq, float* seq_probs, float* seq_score,
                           int* num_finish_beam, int vocab_size, int cur_step, float length_norm,
                           float diverse_lambda, int end_id, int batch_size, int beam_size,
                           int max_step, lsh_stream_t stream);
/* kernels/transformerKernels.h ker_refresh_cache_launcher<int8_t>
 * (transformerKernels.cc.cu:1657-1681): grid_dim_x = decoder layers, grid_dim_y =
 * 2 * batch * beam, block_dim ignored.  self_k_bgeem_offset = bytes between layers. */
int lsh_ker_refresh_cache_i8(int grid_dim_x, int grid_dim_y, int block_dim, lsh_stream_t stream,
                             const int* num_can_per_beam, const int* can_idx,
                             const int8_t* self_k_bgeem, const int8_t* self_v_bgeem,
                             int8_t* new_self_k_bgeem, int8_t* new_self_v_bgeem,
                             int64_t self_k_bgeem_offset, int beam_size, int dim_per_head,
                             int head_num, int vocab_size, int cur_step, int max_step,
                             int diverse, int end_id);
/* kernels/transformerKernels.h ker_write_trg_tokenid_pos_penalty / _neg_penalty /
 * ker_write_topk_result (transformerKernels.cc.cu:1722-1815; launched at
 * model/quant_decoder.cc.cu:454-476 with out_len = cur_step + 1 threads). */
int lsh_ker_write_trg_tokenid_pos_penalty(const int* alive_seq, float* seq_score, int* output,
                                          int max_step, int beam_size, int batch_size,
                                          int out_len, lsh_stream_t stream);
int lsh_ker_write_trg_tokenid_neg_penalty(const int* alive_seq, const float* seq_score,
                                          int* output, int max_step, int beam_size,
                                          int vocab_size, int end_id, int batch_size, int out_len,
                                          lsh_stream_t stream);
int lsh_ker_write_topk_result(const int* alive_seq, float* seq_score, int* res_seq,
                              int vocab_size, int max_step, int beam_size, int end_id,
                              int batch_beam_num, int out_len, lsh_stream_t stream);

/* One whole search step without a sort, a scan or a host round trip: replaces
 * update_new_seq_probs + thrust::sort_by_key + ker_refresh_result of
 * model/quant_decoder.cc.cu:988-1057 (diverse_lambda == 0) and selects the same
 * beams; ties go to the lower candidate id (thrust leaves them unspecified).
 * Workspace: top_score / top_idx [batch*beam, beam_size].  Outputs: new_alive_seq,
 * seq_probs / seq_score (in place), parent [batch*beam] (source beam of each new beam
 * inside its sentence, -1 for a finished beam) and *num_finished. */
int lsh_beam_search_step_i8I_f16(const int8_t* logits, const void* logit_bias, float* seq_probs,
                                 float* seq_score, const int* old_alive_seq, int* new_alive_seq,
                                 float* top_score, int* top_idx, int* parent, int* num_finished,
                                 float dequant_scale, int vocab_size, int max_step,
                                 float length_norm, int cur_step, int batch_size, int beam_size,
                                 int end_id, lsh_stream_t stream);
int lsh_beam_search_step_i8I_f32(const int8_t* logits, const void* logit_bias, float* seq_probs,
                                 float* seq_score, const int* old_alive_seq, int* new_alive_seq,
                                 float* top_score, int* top_idx, int* parent, int* num_finished,
                                 float dequant_scale, int vocab_size, int max_step,
                                 float length_norm, int cur_step, int batch_size, int beam_size,
                                 int end_id, lsh_stream_t stream);
/* The same step with a second workspace, with which the per-row top-k -- bound by vector
 * instructions, one workgroup per row on one compute unit -- is dealt to ceil(vocab_size / 8192)
 * workgroups per row (each computes the row's statistics and the proposals of its part; the
 * merge reads them all).  lsh_beam_search_step_workspace: bytes the shape needs, 0
 * when it does not use one (vocab_size <= 8192, > 32768 or not a multiple of 16).  With a null,
 * short or misaligned (8 bytes) workspace the step runs as lsh_beam_search_step_i8I.  Same
 * beams and ids; the log-sum-exp of a row is added in another order (a last-place difference
 * of the scores).  What QuantTransformer runs.  No counterpart in the reference. */
int64_t lsh_beam_search_step_workspace(int batch_size, int beam_size, int vocab_size);
int lsh_beam_search_step_ws_i8I_f16(const int8_t* logits, const void* logit_bias, float* seq_probs,
                                    float* seq_score, const int* old_alive_seq,
                                    int* new_alive_seq, float* top_score, int* top_idx,
                                    int* parent, int* num_finished, float dequant_scale,
                                    int vocab_size, int max_step, float length_norm, int cur_step,
                                    int batch_size, int beam_size, int end_id, void* workspace,
                                    int64_t workspace_bytes, lsh_stream_t stream);
int lsh_beam_search_step_ws_i8I_f32(const int8_t* logits, const void* logit_bias, float* seq_probs,
                                    float* seq_score, const int* old_alive_seq,
                                    int* new_alive_seq, float* top_score, int* top_idx,
                                    int* parent, int* num_finished, float dequant_scale,
                                    int vocab_size, int max_step, float length_norm, int cur_step,
                                    int batch_size, int beam_size, int end_id, void* workspace,
                                    int64_t workspace_bytes, lsh_stream_t stream);
/* lsh_beam_search_step_i8I_f16 for callers that cannot allocate device memory (code
 * under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  The proposal workspace (top_score / top_idx) is a
 * static device array inside the library, 512 KiB per GPU, so the step is limited to
 * batch_size * beam_size * beam_size <= 65536 (LSH_ERR_UNSUPPORTED beyond); the call
 * allocates and frees nothing.  All calls on one GPU share that GPU's array: calls
 * that overlap in time on one GPU race.  Results are identical to
 * lsh_beam_search_step_i8I_f16. */
int lsh_beam_search_step_noalloc_i8I_f16(const int8_t* logits, const void* logit_bias,
                                         float* seq_probs, float* seq_score,
                                         const int* old_alive_seq, int* new_alive_seq, int* parent,
                                         int* num_finished, float dequant_scale, int vocab_size,
                                         int max_step, float length_norm, int cur_step,
                                         int batch_size, int beam_size, int end_id,
                                         lsh_stream_t stream);
/* Cache reorder driven by the parent table of lsh_beam_search_step_i8I (same copy as
 * lsh_ker_refresh_cache_i8).  rows = batch * beam. */
int lsh_refresh_cache_by_parent_i8(int n_layer, int rows, lsh_stream_t stream, const int* parent,
                                   const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                                   int8_t* v_new, int64_t layer_offset, int beam_size,
                                   int dim_per_head, int head_num, int cur_step, int max_step);

/* ======================================================================== */
/* GPT path                                                                   */
/* ======================================================================== */

/* kernels/gptKernels_int8.h ker_gpt_embedding_i8I_launcher
 * (gptKernels_int8.cc.cu:71-94).  token_emb [vocab, hidden] int8 codes; token_id
 * [batch_size, batch_seq_len]; output [batch_size, batch_seq_len, hidden] T (zeros at
 * padding); real_seq_len[b] += non-padding tokens of row b.  Token ids must lie inside
 * the table, as for the reference. */
int lsh_ker_gpt_embedding_i8I_f16(int batch_size, int batch_seq_len, int hidden_size,
                                  lsh_stream_t stream, const int8_t* token_emb,
                                  const void* pos_emb, const int* token_id, void* output,
                                  int* real_seq_len, int padding_id, int pos_offset,
                                  float dequant_scale);
int lsh_ker_gpt_embedding_i8I_f32(int batch_size, int batch_seq_len, int hidden_size,
                                  lsh_stream_t stream, const int8_t* token_emb,
                                  const void* pos_emb, const int* token_id, void* output,
                                  int* real_seq_len, int padding_id, int pos_offset,
                                  float dequant_scale);
/* The strided-batched int8 GEMM of model/quant_gpt_encoder.cc.cu:498-505:
 * scores[bh, i, j] = sum_d q[bh, i, d] * k[bh, j, d], all [batch*head, seq, ...]. */
int lsh_gpt_scores_i8_i32o(const int8_t* k, const int8_t* q, int32_t* scores, int batch_head_num,
                           int batch_seq_len, int dim_per_head, lsh_stream_t stream);
/* kernels/gptKernels_int8.h ker_correlation_softmax_gpt_i32I_launcher
 * (gptKernels_int8.cc.cu:225-240).  Rows of padded queries (position >= real_seq_len)
 * are written as zeros; the reference leaves them untouched. */
int lsh_ker_correlation_softmax_gpt_i32I_f16(int batch_size, int batch_seq_len, int head_num,
                                             lsh_stream_t stream, const int32_t* correlation,
                                             void* output, const int* real_seq_len,
                                             float attn_scale, float dequant_scale);
int lsh_ker_correlation_softmax_gpt_i32I_f32(int batch_size, int batch_seq_len, int head_num,
                                             lsh_stream_t stream, const int32_t* correlation,
                                             void* output, const int* real_seq_len,
                                             float attn_scale, float dequant_scale);
/* kernels/gptKernels_int8.h ker_arrange_qkv_with_cache_i8I_i8O_launcher
 * (gptKernels_int8.cc.cu:772-798): batch_token_num = batch * batch_seq_len; caches are
 * re-laid out from [batch, head, batch_seq_len-1, d] (k_cache, v_cache) to
 * [batch, head, batch_seq_len, d] (new_k, new_v) with the new token appended. */
int lsh_ker_arrange_qkv_with_cache_i8I_i8O_f16(int batch_token_num, int hidden_size,
                                               lsh_stream_t stream, const int8_t* ori_qkv,
                                               const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                               const int8_t* k_cache, int8_t* new_v,
                                               const int8_t* v_cache, int batch_seq_len,
                                               int dim_per_head, int head_num,
                                               float dequant_scale, float quant_scale,
                                               int in_col32);
int lsh_ker_arrange_qkv_with_cache_i8I_i8O_f32(int batch_token_num, int hidden_size,
                                               lsh_stream_t stream, const int8_t* ori_qkv,
                                               const void* qkv_bias, int8_t* new_q, int8_t* new_k,
                                               const int8_t* k_cache, int8_t* new_v,
                                               const int8_t* v_cache, int batch_seq_len,
                                               int dim_per_head, int head_num,
                                               float dequant_scale, float quant_scale,
                                               int in_col32);
/* kernels/gptKernels_int8.h ker_topk_sample_i8I_launcher (gptKernels_int8.cc.cu:252-463) and
 * ker_topp_sample_i8I_launcher (:465-660).  k == 1: greedy, ties at the maximum go to the lowest
 * token id (racing stores decide in the reference), curandstate unused.  k in {2, 4, 8, 16, 32}
 * and top-p: random sampling as the kernels act with 1024 threads per block (thread t owns the
 * ids congruent to t modulo 1024; at most one candidate per thread at or above the rough k-th
 * largest thread maximum / the nucleus threshold; softmax over the candidates; one uniform
 * number picks the first thread whose cumulative probability reaches it).  Other k ->
 * LSH_ERR_INVALID with the reference's message.  curandstate: in place of the reference's
 * curandState array (seeded with clock(), so no stream of numbers is defined there), an array of
 * lsh_rng_state_t, one per sequence, filled by lsh_rng_setup and advanced by every draw: the
 * uniform number of a draw is word 0 of Philox4x32-10 (key = seed, counter = (draws, 0,
 * sequence, 0)) mapped to (0, 1] as curand_uniform maps 32 bits.  Top-p: the reference reads an
 * uninitialised threshold in all threads but one (:533-539); built is what it intends (the
 * longest prefix of the descending thread maxima whose exp-sum stays within p of the total, at
 * least the largest).  real_seq_len is unused, as in the reference.  vocab_size <= 2^20. */
typedef struct lsh_rng_state {
  uint64_t seed;
  uint32_t sequence, draws;
} lsh_rng_state_t;
/* state[i] = {seed, i, 0} for i < n (replaces ker_curand_setup,
 * kernels/transformerKernels.cc.cu:2270-2274); state 16-byte aligned device memory */
int lsh_rng_setup(void* state, int n, uint64_t seed, lsh_stream_t stream);
int lsh_ker_topk_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len,
                            int max_thread_per_block, lsh_stream_t stream, const int8_t* logits,
                            int* old_input_ids, int* new_input_ids, const int* real_seq_len,
                            int vocab_size, int k, int* unfinished, void* curandstate, int eos_id,
                            float dequant_scale, int in_col32);
int lsh_ker_topp_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len,
                            int max_thread_per_block, lsh_stream_t stream, const int8_t* logits,
                            int* old_input_ids, int* new_input_ids, const int* real_seq_len,
                            int vocab_size, float p, int* unfinished, void* curandstate,
                            int eos_id, float dequant_scale, int in_col32);
/* kernels/transformerKernels_int8.h:123-143 ker_topk_sample_i8I_launcher and
 * ker_topp_sample_i8I_launcher of the encoder-decoder model (bodies
 * transformerKernels_int8.cc.cu:1908-2290; called by QuantDecoder::sample and
 * ::topk_greedy_search, model/quant_decoder.cc.cu:952-998, 1101-1130).  Against the GPT
 * launchers above: a logit is code * dequant_scale + logit_bias[id], the ids live in place in
 * old_input_ids [batch_size, max_step] (column batch_seq_len receives the token; a row whose
 * last token is eos_id gets another eos_id and does not touch the flag), new_input_ids is
 * unused as in the reference.  The fourth-to-last pointer is the "unfinished" word (the
 * reference's header calls it all_finished for top-k): set to 1 when a sampled token is not
 * eos_id; the caller clears it.  k == 1: the first id of the largest logit (a race decides in
 * the reference), curandstate may be null.  Random numbers and the top-p nucleus: as for
 * lsh_ker_topk_sample_i8I above.  The reference's top-p also adds the bias of every id of a
 * thread into that thread's maximum (:2136-2137); built is the maximum of the biased logits. */
int lsh_ker_topk_sample_i8I_dec_f16(int batch_size, int batch_seq_len, int max_step,
                                    int logits_seq_len, int max_thread_per_block,
                                    lsh_stream_t stream, const int8_t* logits,
                                    const void* logit_bias, int* old_input_ids,
                                    int* new_input_ids, int vocab_size, int k, int* all_finished,
                                    void* curandstate, int eos_id, float dequant_scale,
                                    int in_col32);
int lsh_ker_topk_sample_i8I_dec_f32(int batch_size, int batch_seq_len, int max_step,
                                    int logits_seq_len, int max_thread_per_block,
                                    lsh_stream_t stream, const int8_t* logits,
                                    const void* logit_bias, int* old_input_ids,
                                    int* new_input_ids, int vocab_size, int k, int* all_finished,
                                    void* curandstate, int eos_id, float dequant_scale,
                                    int in_col32);
int lsh_ker_topp_sample_i8I_dec_f16(int batch_size, int batch_seq_len, int max_step,
                                    int logits_seq_len, int max_thread_per_block,
                                    lsh_stream_t stream, const int8_t* logits,
                                    const void* logit_bias, int* old_input_ids,
                                    int* new_input_ids, int vocab_size, float p, int* unfinished,
                                    void* curandstate, int eos_id, float dequant_scale,
                                    int in_col32);
int lsh_ker_topp_sample_i8I_dec_f32(int batch_size, int batch_seq_len, int max_step,
                                    int logits_seq_len, int max_thread_per_block,
                                    lsh_stream_t stream, const int8_t* logits,
                                    const void* logit_bias, int* old_input_ids,
                                    int* new_input_ids, int vocab_size, float p, int* unfinished,
                                    void* curandstate, int eos_id, float dequant_scale,
                                    int in_col32);
/* kernels/gptKernels_int8.h:57-61 ker_attention_mask_weights_i32I_launcher
 * (gptKernels_int8.cc.cu:815-853): soft-max of the int32 scores of the last dst_seq_len query
 * positions over src_seq_len <= 1024 keys, query i seeing keys 0 .. i + src_seq_len -
 * dst_seq_len; correlation int32 and output T, both [batch_size, head_num * dst_seq_len,
 * src_seq_len]; rows of queries at or beyond real_seq_len[batch] are left untouched. */
int lsh_ker_attention_mask_weights_i32I_f16(int batch_size, int dst_seq_len, int src_seq_len,
                                            int head_num, lsh_stream_t stream,
                                            const int32_t* correlation, void* output,
                                            const int* real_seq_len, float attn_scale,
                                            float dequant_scale);
int lsh_ker_attention_mask_weights_i32I_f32(int batch_size, int dst_seq_len, int src_seq_len,
                                            int head_num, lsh_stream_t stream,
                                            const int32_t* correlation, void* output,
                                            const int* real_seq_len, float attn_scale,
                                            float dequant_scale);
/* kernels/gptKernels_int8.h ker_ppl_i8I_launcher (gptKernels_int8.cc.cu:182-190). */
int lsh_ker_ppl_i8I(int batch_size, int batch_seq_len, int max_thread_per_block,
                    lsh_stream_t stream, const int8_t* logits, const int* input_ids,
                    const int* real_seq_len, float* ppl, int vocab_size, float dequant_scale,
                    int in_col32);

/* No counterpart in the reference: lsh_ker_ppl_i8I with a workspace of batch_size *
 * batch_seq_len floats, so that every (sequence, position) pair gets its own workgroup and
 * a second kernel adds a sequence's terms in ascending order; the same bits as
 * lsh_ker_ppl_i8I, which walks a sequence's positions in one workgroup (what QuantGpt runs
 * for files with sampling_method "ppl"). */
int lsh_ker_ppl_i8I_workspace(int batch_size, int batch_seq_len, lsh_stream_t stream,
                              const int8_t* logits, const int* input_ids, const int* real_seq_len,
                              float* ppl, int vocab_size, float dequant_scale, float* workspace);

/* Prompt pass of the model, no single counterpart in the reference:
 *  - lsh_gpt_arrange_qkv_prefill_f16 = ker_arrange_encself_qkv_i8I_i8O_launcher
 *    (model/quant_gpt_encoder.cc.cu:489-496) writing q / k as fp16 code values and v
 *    dequantised, each [batch, head, seq, d], plus k / v codes into caches of fixed
 *    stride [batch, head, max_step, d];
 *  - lsh_gpt_prefill_attention_f16 = the int8 q.K^T GEMM, ker_correlation_softmax_gpt_i32I,
 *    the P.V GEMM and ker_arrange_atten_output_i8O (:498-530) in one causal kernel: the
 *    fp32 MFMA accumulators over code values are the exact int32 scores.  ctx
 *    ([batch, head, seq, d] fp16) and ctx_q ([batch*seq, hidden] int8) are each optional;
 *  - lsh_gpt_greedy_step = ker_topk_sample_i8I<1> on ids kept in place as
 *    [batch, max_step]: writes column cur_len, last_ids[batch] and the unfinished flag;
 *  - lsh_gpt_sample_step = ker_topk_sample_i8I<k> (k in {2, 4, 8, 16, 32}) or, with k == 0,
 *    ker_topp_sample_i8I with p, on the same in-place ids; state as for
 *    lsh_ker_topk_sample_i8I. */
int lsh_gpt_arrange_qkv_prefill_f16(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                    const int8_t* ori_qkv, const void* qkv_bias, void* q_codes,
                                    void* k_codes, void* v_deq, int8_t* k_cache, int8_t* v_cache,
                                    int batch_seq_len, int dim_per_head, int head_num,
                                    int max_step, float dequant_scale, float quant_scale);
int lsh_gpt_prefill_attention_f16(const void* q_codes, const void* k_codes, const void* v,
                                  const int* real_seq_len, void* ctx, int8_t* ctx_q,
                                  float quant_scale, float dequant_scale, int batch_size,
                                  int batch_seq_len, int head_num, int dim_per_head,
                                  lsh_stream_t stream);
/* The same two stages on int8 codes end to end (no counterpart in the reference; what QuantGpt
 * runs for heads of 64 and prompts of at most 1024 tokens -- lsh_gpt_prefill_i8_supported):
 *  - lsh_gpt_arrange_qkv_prefill_i8 = ker_arrange_encself_qkv_i8I_i8O_launcher
 *    (model/quant_gpt_encoder.cc.cu:489-496) writing the requantised q codes
 *    [batch, head, seq, d] and the k / v codes straight into the caches
 *    [batch, head, max_step, d]; nothing is written as fp16.  hidden % 128 == 0, head size 16,
 *    32, 64 or a multiple of 128;
 *  - lsh_gpt_prefill_attention_i8 = the q.K^T GEMM on the codes (int32 scores, bit for bit),
 *    ker_correlation_softmax_gpt_i32I, the P.V GEMM over values half(code / v_quant_scale) (what
 *    the arrange kernel of the reference stores as dequantised v) and
 *    ker_arrange_atten_output_i8O (:498-530) in one causal kernel that reads the q codes and
 *    the caches; ctx_q [batch * seq, hidden] int8; queries at or beyond real_seq_len give
 *    zeros.  dequant_scale dequantises q and k codes (scores = int32 * attn_scale *
 *    dequant_scale^2). */
int lsh_gpt_prefill_i8_supported(int batch_seq_len, int head_num, int dim_per_head);
/* Process-wide switch: QuantGpt's prompt pass on the int8 codes where the shape is covered
 * (default) or through the fp16-storage pair above; returns the previous setting.  The two
 * routes give the same bytes. */
int lsh_gpt_prefill_on_codes_in_models(int on);
int lsh_gpt_arrange_qkv_prefill_i8(int batch_token_num, int hidden_size, lsh_stream_t stream,
                                   const int8_t* ori_qkv, const void* qkv_bias, int8_t* q_codes,
                                   int8_t* k_cache, int8_t* v_cache, int batch_seq_len,
                                   int dim_per_head, int head_num, int max_step,
                                   float dequant_scale, float quant_scale);
int lsh_gpt_prefill_attention_i8(const int8_t* q_codes, const int8_t* k_cache,
                                 const int8_t* v_cache, const int* real_seq_len, int8_t* ctx_q,
                                 float quant_scale, float dequant_scale, float v_quant_scale,
                                 int batch_size, int batch_seq_len, int head_num, int dim_per_head,
                                 int max_step, lsh_stream_t stream);
int lsh_gpt_greedy_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size,
                        int max_step, int cur_len, int batch_size, int* unfinished, int eos_id,
                        lsh_stream_t stream);
int lsh_gpt_sample_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size,
                        int max_step, int cur_len, int batch_size, int* unfinished, int eos_id,
                        int k, float p, float dequant_scale, void* state, lsh_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LIGHTSEQ_HIP_H_ */
