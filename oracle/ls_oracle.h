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
  const float* clip_max;          /* [n_layer * 11], proto/quant_bert_weight.cc:194-205 */
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

#ifdef __cplusplus
}
#endif
#endif /* LS_ORACLE_H_ */
