/*
 * CPU oracle for the int8 transformer-layer forward path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * algorithm; only the test-suite, the smoke check and the cpu_baseline leg of
 * the benchmark may link or call it.  Nothing in the shipped library does.
 *
 * Conventions
 *  - `f16` selects the storage type T of activations / biases / LN parameters:
 *    1 = IEEE binary16 stored as uint16_t bit patterns, 0 = float.
 *  - Every reduction (LayerNorm mean / variance, softmax sum, attention dot
 *    products) is accumulated in double and rounded once to float: the
 *    reference reduces in float with a block-tree order that no sequential loop
 *    reproduces, and the double sum is the centre of all such orders.
 *  - All other arithmetic is float, in the order the reference writes it,
 *    compiled with -ffp-contract=off.
 *
 * Citations are to files below lightseq/inference/ of the reference unless
 * they start with csrc/.
 */
#ifndef LS_ORACLE_H_
#define LS_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- binary16 helpers ---------------------------------------------------- */
float lso_h2f(uint16_t h);
uint16_t lso_f2h(float f); /* round-to-nearest-even, like __float2half_rn */

/* ---- scalar quantisers: kernels/transformerKernels_int8.cc.cu:14-27 ------- */
int8_t lso_float2int8(float x, float quant_scale);
int8_t lso_posfloat2int8(float x, float quant_scale, float clip_max);

/* kernels/transformerKernels_int8.cc.cu:29-82 */
void lso_quantize_tensor(const void* in, int8_t* out, long n, float quant_scale,
                         int f16);
/* kernels/transformerKernels_int8.cc.cu:84-147 */
void lso_dequantize_tensor(const int32_t* in, void* out, long n,
                           float dequant_scale, int f16);

/* kernels/transformerKernels_int8.cc.cu:149-316 */
void lso_norm_layer_resual_i8O(void* input, int8_t* output, const void* scale,
                               const void* bias, const void* residual_bias,
                               int tokens, int hidden, float quant_scale,
                               int is_post_ln, int f16);

/* kernels/transformerKernels_int8.cc.cu:318-705 (in_is_i32 picks the i32I /
 * i8I variant) */
void lso_residual_bias_ln_i8O(const void* input, int in_is_i32,
                              const void* scale, const void* bias,
                              const void* residual_bias, int8_t* output,
                              void* residual, int tokens, int hidden,
                              float dequant_scale, float quant_scale,
                              int is_post_ln, const void* colsum, int f16);

/* kernels/transformerKernels_int8.cc.cu:707-863 */
void lso_residual_bias_ln_i32I(const int32_t* input, const void* scale,
                               const void* bias, const void* residual,
                               void* output, int tokens, int hidden,
                               float dequant_scale, const void* colsum,
                               int f16);

/* kernels/transformerKernels_int8.cc.cu:865-964, kernels/common.h:17-23 */
void lso_bias_gelu_i8I_i8O(const int8_t* input, int8_t* output,
                           const void* bias, int tokens, int feature_dim,
                           float dequant_scale, float quant_scale, int f16);
/* kernels/transformerKernels_int8.cc.cu:966-1078 */
void lso_bias_relu_i8I_i8O(const int8_t* input, int8_t* output,
                           const void* bias, int tokens, int feature_dim,
                           float dequant_scale, float quant_scale,
                           float clip_max, int narrow_clip, int f16);

/* kernels/transformerKernels_int8.cc.cu:1080-1183.  new_qkv holds q at 0,
 * k at max_batch_dim, v at 2*max_batch_dim, each [B,h,S,d]. */
void lso_arrange_encself_qkv_i8I(const int8_t* ori_qkv, const void* qkv_bias,
                                 void* new_qkv, long max_batch_dim, int batch,
                                 int seq_len, int dim_per_head, int head_num,
                                 float dequant_scale, int f16);
/* kernels/transformerKernels_int8.cc.cu:1185-1299 */
void lso_arrange_encself_qkv_i8I_i8O(const int8_t* ori_qkv,
                                     const void* qkv_bias, int8_t* new_q,
                                     int8_t* new_k, int8_t* new_v, void* d_v,
                                     int batch, int seq_len, int dim_per_head,
                                     int head_num, float dequant_scale,
                                     float quant_scale, int f16);
/* kernels/transformerKernels_int8.cc.cu:1301-1393 ([B,h,S,d] -> [B*S,H] i8) */
void lso_arrange_atten_output_i8O(const void* ori_q, int8_t* new_q, int tokens,
                                  int beam_size, int dim_per_head, int head_num,
                                  float quant_scale, int f16);

/* kernels/transformerKernels.cc.cu:1119-1172 */
void lso_correlation_softmax_encself(void* correlation, const int* pad_mask,
                                     int batch, int seq_len, int head_num,
                                     int f16);

/* model/quant_bert_encoder.cc.cu:321-341: the two strided-batched attention
 * GEMMs.  scores[b,h,i,j] = T(alpha * sum_d q[b,h,i,d] k[b,h,j,d]) with alpha
 * first rounded to T; ctx[b,h,i,d] = T(sum_j p[b,h,i,j] v[b,h,j,d]). */
void lso_attn_scores(const void* q, const void* k, void* scores, int batch_heads,
                     int seq_len, int dim_per_head, float alpha, int f16);
void lso_attn_context(const void* probs, const void* v, void* ctx,
                      int batch_heads, int seq_len, int dim_per_head, int f16);

/* model/cublas_helper.cc:361-489.  A [M,K], W [N,K] (both K-contiguous),
 * C [M,N] row-major. */
void lso_gemm_i8_i32(const int8_t* A, const int8_t* W, int32_t* C, int M, int N,
                     int K);
/* int8 output: clamp(floor(float(acc)*alpha + 0.5), -127, 127) -- the rounding
 * of the closed-source cuBLASLt epilogue is not defined by any reference file;
 * this is the north-star rule with the repository's tie rule. */
void lso_gemm_i8_i8(const int8_t* A, const int8_t* W, int8_t* C, int M, int N,
                    int K, float alpha);
int8_t lso_requant_acc(int32_t acc, float alpha);

/* kernels/embKernels_int8.cc.cu:13-155 */
void lso_enc_emb_i8I(const int8_t* token_emb, const void* pos_emb,
                     const int* tokens, void* output, int* pad_mask, int pad_id,
                     int batch, int seq_len, int hidden, float dequant_scale,
                     int scaled, int f16);
/* kernels/transformerKernels.cc.cu:18-80: out[c] = T(scale * sum_r inp[r,c]) */
void lso_scaled_colsum(const void* inp, void* out, int rows, int cols,
                       float scale, int f16);

/* ---- whole encoder stack: model/quant_bert_encoder.cc.cu:214-520 ---------- */
typedef struct {
  int n_layer, hidden, inner, head_num, max_step, vocab, padding_id;
  int is_post_ln, use_gelu;
  int f16; /* storage type of all T-typed arrays below */
  /* embedding */
  const int8_t* tok_emb_q; /* [vocab, hidden] int8 codes */
  const void* pos_emb;     /* [max_step, hidden] */
  const void* final_ln_scale;
  const void* final_ln_bias;
  float emb_clip_max;
  /* per layer (arrays of n_layer pointers) */
  const void* const* ln1_scale;
  const void* const* ln1_bias;
  const int8_t* const* w_qkv; /* [3H, H] int8 codes, K-contiguous */
  const void* const* b_qkv;
  const int8_t* const* w_out; /* [H, H] */
  const void* const* b_out;
  const void* const* ln2_scale;
  const void* const* ln2_bias;
  const int8_t* const* w_ffn1; /* [I, H] */
  const void* const* b_ffn1;
  const int8_t* const* w_ffn2; /* [H, I] */
  const void* const* b_ffn2;
  const void* const* ffn2_colsum; /* [H] or NULL entries (GELU) */
  const float* clip_max;          /* [n_layer * clip_stride], proto/quant_bert_weight.cc:194-205 */
  /* 11 / 0 for QuantBert; 12 / 1 for the encoder of QuantTransformer
   * (model/quant_encoder.cc.cu:140, :242; proto/quant_transformer_weight.cc:316-328) */
  int clip_stride;
  int emb_scaled;
} lso_bert_weights;

/* Optional taps: when non-NULL, receive a copy of the named intermediate of
 * layer `tap_layer` (sizes in comments, M = batch*seq_len). */
typedef struct {
  int tap_layer;
  int8_t* ln1_q;     /* [M,H]   input of the QKV GEMM */
  int8_t* qkv_q;     /* [M,3H]  QKV GEMM output */
  void* ctx;         /* [B,h,S,d] attention context (T) */
  int8_t* ctx_q;     /* [M,H]   input of the out-proj GEMM */
  int8_t* out_q;     /* [M,H]   out-proj GEMM output */
  int8_t* ln2_q;     /* [M,H]   input of FFN1 */
  int8_t* ffn1_q;    /* [M,I]   FFN1 GEMM output */
  int8_t* act_q;     /* [M,I]   input of FFN2 */
  int32_t* ffn2_acc; /* [M,H]   FFN2 accumulators */
} lso_bert_taps;

/* Returns 0 on success, non-zero on a violated precondition. */
int lso_quant_bert_encoder(const lso_bert_weights* w, const int* token_ids,
                           int batch, int seq_len, void* output /*[M,H] T*/,
                           int* pad_mask /*[M]*/, const lso_bert_taps* taps);

/* ========================================================================= */
/* decoder half                                                                */
/* ========================================================================= */

/* kernels/embKernels_int8.cc.cu:158-200.  tokens [rows, max_step]; token_emb is
 * [hidden, vocab] as the reference stores it (vocab_major = 0) or [vocab, hidden]
 * (vocab_major = 1, the table of the logits GEMM); output [rows, hidden] T. */
void lso_dec_emb_i8I(const int8_t* token_emb, const void* pos_emb,
                     const int* tokens, void* output, int rows, int hidden,
                     int vocab, int step, int max_step, float dequant_scale,
                     int scaled, int vocab_major, int f16);

/* kernels/transformerKernels_int8.cc.cu:1395-1499.  ori_qkv [rows, 3H] int8;
 * new_q [rows, H]; caches [rows, head_num, max_step, dim_per_head] int8. */
void lso_arrange_decself_qkv_i8I_i8O(const int8_t* ori_qkv, const void* qkv_bias,
                                     int8_t* new_q, int8_t* k_cache,
                                     int8_t* v_cache, int rows, int head_num,
                                     int dim_per_head, int max_step, int step_id,
                                     float dequant_scale, float quant_scale,
                                     int f16);

/* model/quant_decoder.cc.cu:676-683 (strided-batched int8 GEMM):
 * scores[r*head_num+h, j] = sum_d q[r,h,d] * k_cache[r,h,j,d], j < step_num;
 * row stride of scores is max_step. */
void lso_decself_scores(const int8_t* q, const int8_t* k_cache, int32_t* scores,
                        int rows, int head_num, int dim_per_head, int max_step,
                        int step_num);

/* kernels/transformerKernels_int8.cc.cu:1515-1594 */
void lso_fuse_softmax_new_value_i32I_i8O(const int32_t* logits, const int8_t* v,
                                         int8_t* new_v, int batch_head_num,
                                         int step_num, int max_step, int head_num,
                                         int dim_per_head, float attn_scale,
                                         float dequant_scale, float quant_scale);

/* kernels/transformerKernels_int8.cc.cu:1596-1688.  new_q [batch, head_num,
 * beam_size, dim_per_head] T. */
void lso_arrange_encdec_q_i8I(const int8_t* ori_q, const void* q_bias, void* new_q,
                              int rows, int beam_size, int dim_per_head,
                              int head_num, float dequant_scale, int f16);

/* kernels/transformerKernels.cc.cu:903-1020.  ori_kv [tokens, n_layer, 2, H] T;
 * new_k / new_v: layer l at element offset l*offset_per_layer, laid out
 * [batch, head_num, seq_len, dim_per_head]. */
void lso_arrange_encdec_kv(const void* ori_kv, const void* kv_bias, void* new_k,
                           void* new_v, long offset_per_layer, int batch,
                           int seq_len, int n_layer, int dim_per_head,
                           int head_num, int f16);

/* kernels/transformerKernels.cc.cu:1226-1284.  correlation [batch,
 * head_num*beam_size, seq_len] T, in place. */
void lso_correlation_softmax_encdec(void* correlation, const int* pad_mask,
                                    int batch, int heads_x_beams, int seq_len,
                                    int f16);

/* model/quant_decoder.cc.cu:767-790: rectangular versions of the two attention
 * GEMMs (n_q queries against n_k keys per batch-head). */
void lso_attn_scores_rect(const void* q, const void* k, void* scores,
                          int batch_heads, int n_q, int n_k, int dim_per_head,
                          float alpha, int f16);
void lso_attn_context_rect(const void* probs, const void* v, void* ctx,
                           int batch_heads, int n_q, int n_k, int dim_per_head,
                           int f16);

/* model/quant_decoder.cc.cu:497-501: C[M,N] = T(A[M,K] @ B[K,N]), T operands. */
void lso_gemm_T(const void* A, const void* B, void* C, int M, int N, int K, int f16);

/* kernels/transformerKernels.h:137-140 */
float lso_length_norm(int length, float alpha);

/* kernels/transformerKernels_int8.cc.cu:1690-1890 with diverse_lambda == 0.
 * Candidates are emitted row by row in ascending vocabulary order (the reference
 * emits the same set in an order decided by atomics).  num_beam_can[0] = total,
 * num_beam_can[1 + row] = candidates of that row.  Returns the total. */
int lso_select_beam_rough_topk_i8I(const int8_t* logits, const void* logit_bias,
                                   const float* seq_probs, const float* seq_score,
                                   const int* alive_seq, float dequant_scale,
                                   int* can_idx, float* can_score,
                                   int* num_beam_can, int vocab_size, int max_step,
                                   float length_norm, int cur_step,
                                   int step_token_num, int max_thread_per_block,
                                   int beam_size, int end_id, int f16);

/* thrust::exclusive_scan + thrust::sort_by_key(greater) of
 * model/quant_decoder.cc.cu:1002-1003 and :1095-1096; ties keep emission order
 * (thrust leaves them unspecified). */
void lso_scan_sort_candidates(int* can_idx, float* can_score, int* num_beam_can,
                              int step_token_num);

/* kernels/transformerKernels.cc.cu:1398-1463 with diverse_lambda == 0.
 * num_can_per_beam is the scanned array (num_beam_can + 1). */
void lso_refresh_result(const int* can_idx, const float* can_score,
                        const int* num_can_per_beam, const int* old_alive_seq,
                        int* new_alive_seq, float* seq_probs, float* seq_score,
                        int* num_finish_beam, int vocab_size, int cur_step,
                        float length_norm, int end_id, int batch, int beam_size,
                        int max_step);

/* kernels/transformerKernels.cc.cu:1579-1627 (int8 cache).  Caches hold n_layer
 * blocks of cache_offset bytes, each [rows, head_num, max_step, dim_per_head]. */
void lso_refresh_cache_i8(const int* num_can_per_beam, const int* can_idx,
                          const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                          int8_t* v_new, long cache_offset, int n_layer, int batch,
                          int beam_size, int dim_per_head, int head_num,
                          int vocab_size, int cur_step, int max_step, int end_id);

/* kernels/transformerKernels.cc.cu:1707-1815.  out_len = cur_step + 1. */
void lso_write_trg_tokenid_pos_penalty(const int* alive_seq, float* seq_score,
                                       int* output, int max_step, int beam_size,
                                       int batch, int out_len);
void lso_write_trg_tokenid_neg_penalty(const int* alive_seq, const float* seq_score,
                                       int* output, int max_step, int beam_size,
                                       int end_id, int batch, int out_len);
void lso_write_topk_result(const int* alive_seq, float* seq_score, int* res_seq,
                           int max_step, int beam_size, int end_id, int rows,
                           int out_len);

/* ---- whole decoder: model/quant_decoder.cc.cu:413-1075 -------------------- */
typedef struct {
  int n_layer, hidden, inner, head_num, max_step, vocab;
  int beam_size, extra_decode_length, start_id, end_id;
  int is_post_ln, use_gelu, f16;
  float length_penalty;
  const int8_t* tok_emb_q;      /* [vocab, hidden] int8 codes */
  const void* pos_emb;          /* [max_step, hidden] */
  const void* out_ln_scale;     /* trg_embedding.norm_scale */
  const void* out_ln_bias;
  const void* encdec_kv_kernel; /* [hidden, n_layer*2*hidden] T (dequantised) */
  const void* encdec_kv_bias;   /* [n_layer, 2, hidden] */
  const void* logit_bias;       /* [vocab] */
  float emb_clip_max, output_ln_clip_max, logits_clip_max;
  /* per layer (arrays of n_layer pointers); int8 kernels are [N, K] codes */
  const void* const* self_ln_scale;
  const void* const* self_ln_bias;
  const int8_t* const* w_self_qkv;
  const void* const* b_self_qkv;
  const int8_t* const* w_self_out;
  const void* const* b_self_out;
  const void* const* encdec_ln_scale;
  const void* const* encdec_ln_bias;
  const int8_t* const* w_encdec_q;
  const void* const* b_encdec_q;
  const int8_t* const* w_encdec_out;
  const void* const* b_encdec_out;
  const void* const* ffn_ln_scale;
  const void* const* ffn_ln_bias;
  const int8_t* const* w_ffn1;
  const void* const* b_ffn1;
  const int8_t* const* w_ffn2;
  const void* const* b_ffn2;
  const void* const* ffn2_colsum; /* NULL (GELU) or n_layer [H] arrays */
  const float* clip_max;          /* [n_layer * 19], proto/quant_transformer_weight.cc:490-508 */
} lso_dec_weights;

typedef struct {
  /* forced_logits: when non-NULL, step t's search consumes
   * forced_logits[t] ([rows, vocab] int8) instead of the oracle's own logits, so
   * the token history follows the run that produced them. */
  const int8_t* forced_logits;
  int forced_steps;
  int8_t* logits_record;  /* NULL or [max_step, rows, vocab]: the oracle's own logits */
  int* alive_seq_record;  /* NULL or [max_step, rows, max_step]: alive_seq after each step */
  float* seq_probs_record; /* NULL or [max_step, rows] */
  int steps_run;          /* out: number of run_step calls */
  int early_stopped;      /* out */
} lso_dec_trace;

/* Beam search (sampling_method "beam_search", diverse_lambda 0).  enc_out
 * [batch, seq_len, hidden] T, pad_mask [batch, seq_len].
 * output_topk = 0: result [batch, *out_len], scores [batch] (first `batch` slots
 * of the score array, as the reference leaves them);
 * output_topk = 1 (what pywrapper/quant_transformer.cc:51-53 passes): result
 * [batch*beam, *out_len], scores [batch*beam]; the score of a beam that never
 * finished is whatever the score buffer held (0 here).
 * `is_benchmark` reproduces benchmark_mode(true): no early stop.
 * Returns 0 on success. */
int lso_quant_decoder(const lso_dec_weights* w, const void* enc_out,
                      const int* pad_mask, int batch, int seq_len, int is_benchmark,
                      int output_topk, int* result, int* out_len, float* scores,
                      lso_dec_trace* trace);

/* ========================================================================= */
/* GPT half (ls_oracle_gpt.c)                                                  */
/* ========================================================================= */

/* kernels/gptKernels_int8.cc.cu:21-106.  token_emb [vocab, hidden]; token_id
 * [batch, seq_len]; real_seq_len[b] += number of non-padding tokens of row b. */
void lso_gpt_embedding_i8I(const int8_t* token_emb, const void* pos_emb,
                           const int* token_id, void* output, int* real_seq_len,
                           int padding_id, int pos_offset, float dequant_scale,
                           int batch, int seq_len, int hidden, int f16);

/* model/quant_gpt_encoder.cc.cu:498-505: scores[bh, i, j] = sum_d q[bh,i,d] k[bh,j,d] */
void lso_gpt_scores_i8(const int8_t* q, const int8_t* k, int32_t* scores,
                       int batch_heads, int seq_len, int dim_per_head);

/* kernels/gptKernels_int8.cc.cu:192-250.  Rows of padded queries are written as
 * zeros (the reference leaves them untouched). */
/* ker_attention_mask_weights_i32I (gptKernels_int8.cc.cu:815-843) */
void lso_attention_mask_weights_i32I(const int32_t* correlation, void* output,
                                     const int* real_seq_len, int batch, int dst_seq_len,
                                     int src_seq_len, int head_num, float attn_scale,
                                     float dequant_scale, int f16);
void lso_correlation_softmax_gpt_i32I(const int32_t* correlation, void* output,
                                      const int* real_seq_len, int batch,
                                      int seq_len, int head_num, float attn_scale,
                                      float dequant_scale, int f16);

/* kernels/gptKernels_int8.cc.cu:658-812: one new token per sequence; the caches
 * are re-laid out from [batch, head, seq_len-1, d] to [batch, head, seq_len, d]
 * with the new key / value appended; new_q [batch, head, 1, d]. */
void lso_arrange_qkv_with_cache_i8I_i8O(const int8_t* ori_qkv, const void* qkv_bias,
                                        int8_t* new_q, int8_t* new_k,
                                        const int8_t* k_cache, int8_t* new_v,
                                        const int8_t* v_cache, int batch,
                                        int seq_len, int dim_per_head,
                                        int head_num, float dequant_scale,
                                        float quant_scale, int f16);

/* kernels/gptKernels_int8.cc.cu:252-463 with k == 1 (greedy).  old ids
 * [batch, seq_len] -> new ids [batch, seq_len + 1]; the sampled ids are also
 * stored behind the old array (old_input_ids[batch*seq_len + b]); a sequence whose
 * last token is eos_id gets eos_id again.  Ties at the maximum go to the lowest
 * token id (the reference lets racing stores decide).  *unfinished is set to 1
 * when any freshly sampled token differs from eos_id. */
void lso_topk_sample_i8I_greedy(const int8_t* logits, int* old_input_ids,
                                int* new_input_ids, int vocab_size, int batch,
                                int seq_len, int logits_seq_len, int* unfinished,
                                int eos_id, float dequant_scale);

/* kernels/gptKernels_int8.cc.cu:108-190.  logits [batch, seq_len, vocab]; ppl[b] +=
 * mean negative log-likelihood of tokens 1 .. real_seq_len-1. */
void lso_ppl_i8I(const int8_t* logits, const int* input_ids, const int* real_seq_len,
                 float* ppl, int vocab_size, float dequant_scale, int batch,
                 int seq_len);

/* ---- whole model: model/quant_gpt_encoder.cc.cu:253-824 ------------------- */
typedef struct {
  int n_layer, hidden, inner, head_num, max_step, vocab, padding_id, eos_id;
  int extra_decode_length, f16;
  const int8_t* tok_emb_q; /* [vocab, hidden] codes */
  const void* pos_emb;
  const void* out_ln_scale;
  const void* out_ln_bias;
  float emb_clip_max, output_ln_clip_max, logits_clip_max;
  const void* const* ln1_scale;
  const void* const* ln1_bias;
  const int8_t* const* w_qkv;
  const void* const* b_qkv;
  const int8_t* const* w_out;
  const void* const* b_out;
  const void* const* ln2_scale;
  const void* const* ln2_bias;
  const int8_t* const* w_ffn1;
  const void* const* b_ffn1;
  const int8_t* const* w_ffn2;
  const void* const* b_ffn2;
  const float* clip_max; /* [n_layer * 12], proto/quant_gpt_weight.cc:228-240 */
} lso_gpt_weights;

/* sampling_method "ppl": ppl [batch].  Returns 0 on success. */
int lso_quant_gpt_ppl(const lso_gpt_weights* w, const int* token_ids, int batch,
                      int seq_len, float* ppl);
/* sampling_method "topk" with topk == 1.  out_ids [batch, *out_len].
 * logits_record: NULL or [max_step, batch, vocab] (the logits of the last position at
 * every sampling step); forced_logits likewise replaces the oracle's own logits in the
 * arg-max for the first forced_steps steps.  *steps_run counts sampling steps. */
int lso_quant_gpt_sample(const lso_gpt_weights* w, const int* token_ids, int batch,
                         int seq_len, int is_benchmark, int* out_ids, int* out_len,
                         const int8_t* forced_logits, int forced_steps,
                         int8_t* logits_record, int* steps_run);

#ifdef __cplusplus
}
#endif
#endif /* LS_ORACLE_H_ */
