// Host-side internal interface between the kernel translation units and the
// C ABI (capi.cpp).  Every function returns an LSH_* status and records a message
// retrievable through lsh_last_error().
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cmath>
#include <mutex>
#include <string>

#include "../../include/lightseq_hip.h"

namespace lsh {

// Records `msg` as the calling thread's last error and returns `code`.
int lsh_fail(int code, const char* msg);
// hipGetLastError() after a launch -> status.
int lsh_check_launch(const char* what);
int lsh_check_hip(hipError_t e, const char* what);

// ---- quantise / dequantise (quant_kernels.hip) -------------------------------
template <typename T>
int quantize_tensor(const T* input, int8_t* output, long n, float quant_scale, hipStream_t s);
template <typename T>
int dequantize_tensor(const int32_t* input, T* output, long n, float dequant_scale,
                      hipStream_t s);
// rows x cols T (row-major) -> int8 codes, optionally transposed to cols x rows
template <typename T>
int quantize_transpose(const T* input, int8_t* output, int rows, int cols, float quant_scale,
                       bool transpose, hipStream_t s);
// stored uint8 (= code + 127) kernels -> int8 codes (optionally transposed) / T values
// p[0..n) = value by a kernel (graph-capture safe, unlike hipMemsetAsync here)
int fill_i32(int* p, int value, int n, hipStream_t s);
int stored_u8_to_i8(const uint8_t* input, int8_t* output, int rows, int cols, bool transpose,
                    hipStream_t s);
template <typename T>
int stored_u8_dequant(const uint8_t* input, T* output, long n, float clip_max, hipStream_t s);
template <typename T>
int scaled_colsum(const T* inp, T* out, int rows, int cols, float scale, hipStream_t s);

// ---- bias + activation + requant (act_kernels.hip) -----------------------------
template <typename T>
int bias_gelu_i8I_i8O(int tokens, hipStream_t s, const int8_t* input, int8_t* output,
                      const T* bias, int feature_dim, float dequant_scale, float quant_scale);
template <typename T>
int bias_relu_i8I_i8O(int tokens, hipStream_t s, const int8_t* input, int8_t* output,
                      const T* bias, int feature_dim, float dequant_scale, float quant_scale,
                      float clip_max, bool narrow_clip);

// ---- LayerNorm family (ln_kernels.hip) ------------------------------------------
template <typename T>
int norm_layer_resual_i8O(int token_num, int hidden_size, hipStream_t stream, T* input,
                          int8_t* output, const T* scale, const T* bias, const T* residual_bias,
                          float quant_scale, bool is_post_ln);
// launch_dec_emb_i8I (vocabulary-major table) followed by norm_layer_resual_i8O under an
// LnFewRowsScope, in one launch: residual receives what the layer norm leaves there, out_q its
// int8 codes.  hidden % 4 == 0, hidden <= 1024.
template <typename T>
int gpt_emb_step_norm_layer_i8O(const int8_t* token_emb, const T* pos_emb, const int* token_id,
                                T* residual, int8_t* out_q, const T* scale, const T* bias,
                                const T* residual_bias, int* real_seq_len, int* zero_flag,
                                int batch_size, int hidden, int vocab, int padding_id, int pos,
                                int max_step, float dequant_scale, float quant_scale,
                                bool is_post_ln, hipStream_t s);
template <typename T>
int dec_emb_norm_layer_i8O(const int8_t* token_emb, const T* pos_emb, const int* tokens,
                           T* residual, int8_t* out_q, const T* scale, const T* bias,
                           const T* residual_bias, int rows, int hidden, int vocab, int step,
                           int max_step, float dequant_scale, bool scaled, float quant_scale,
                           bool is_post_ln, hipStream_t s);
template <typename T, typename AccT>
int residual_bias_ln_i8O(const AccT* input, const T* scale, const T* bias, const T* residual_bias,
                         int8_t* output, T* residual, int batch_tokens, int hidden_size,
                         float dequant_scale, float quant_scale, hipStream_t stream,
                         bool is_post_ln, const T* colsum, int nparts = 1, long part_stride = 0);
template <typename T>
int residual_bias_ln_i32I(const int32_t* input, const T* scale, const T* bias, const T* residual,
                          T* output, int batch_tokens, int hidden_size, float dequant_scale,
                          hipStream_t stream, const T* colsum, int nparts = 1,
                          long part_stride = 0);
// `nparts` > 1: `input` holds that many int32 accumulator planes `part_stride` elements apart
// (split-K GEMM output, gemm_i8_i32o_splitk) which are summed before the dequantisation.
//
// While an object of this type lives, the calling thread's layer-norm launches (hidden <=
// 1024, aligned operands) use the workgroup-per-row kernel, whose small code starts faster
// on launches of a few rows.  It sums a row in another order than the default kernel, so a
// caller keeps one choice for all launches whose results it compares (the decode-step
// loops hold it for every step).
struct LnFewRowsScope {
  LnFewRowsScope();
  ~LnFewRowsScope();
  LnFewRowsScope(const LnFewRowsScope&) = delete;
  LnFewRowsScope& operator=(const LnFewRowsScope&) = delete;

 private:
  bool _prev;
};
// The same switch without a scope (returns the previous setting).
bool ln_set_few_rows(bool on);

// ---- head split / merge, embedding (arrange_kernels.hip) -------------------------
template <typename T>
int arrange_encself_qkv_i8I(int batch_token_num, int hidden_size, hipStream_t s,
                            const int8_t* ori_qkv, const T* qkv_bias, T* new_qkv,
                            long max_batch_dim, int batch_seq_len, int dim_per_head, int head_num,
                            float dequant_scale);
template <typename T>
int arrange_encself_qkv_i8I_i8O(int batch_token_num, int hidden_size, hipStream_t s,
                                const int8_t* ori_qkv, const T* qkv_bias, int8_t* new_q,
                                int8_t* new_k, int8_t* new_v, T* d_v, int batch_seq_len,
                                int dim_per_head, int head_num, float dequant_scale,
                                float quant_scale);
template <typename T>
int arrange_atten_output_i8O(int batch_token_num, int hidden_size, hipStream_t s, const T* ori_q,
                             int8_t* new_q, int beam_size, int dim_per_head, int head_num,
                             float quant_scale);
// vocab_size > 0 clamps the token ids into the table; <= 0 uses them unchecked
template <typename T>
int enc_emb_i8I(const int8_t* token_emb, const T* pos_emb, const int* tokens, T* output,
                int* pad_mask, int pad_id, int batch_size, int seq_len, int hidden_dim,
                hipStream_t s, float dequant_scale, bool scaled, int vocab_size);

// ---- out-projection GEMM + residual LayerNorm in one kernel (ln_kernels.hip) -------------
// [N, K] int8 -> the 16-row x 64-byte MFMA-ordered tiling the fused kernel streams
int tile_weight_16x64(const int8_t* w, int8_t* tiled, int N, int K, hipStream_t s);
bool gemm_ln_fused_supported(int hidden, int K);
// the next fused launch of this thread records its own begin / end timestamps into the events
void gemm_ln_time_next_launch(hipEvent_t start, hipEvent_t stop);
// output / residual as residual_bias_ln_i8O would leave them after gemm_i8_i8o(A, W, alpha)
template <typename T>
int gemm_i8_residual_ln_i8O(const int8_t* A, const int8_t* w_tiled, float alpha, const T* scale,
                            const T* bias, const T* residual_bias, int8_t* output, T* residual,
                            int batch_tokens, int hidden_size, int K, float dequant_scale,
                            float quant_scale, hipStream_t stream, bool is_post_ln);

// ---- encoder attention (attn_kernels.hip) ------------------------------------------
template <typename T>
int correlation_softmax_encself(int batch_size, int batch_seq_len, int head_num, hipStream_t s,
                                T* correlation, const int* src_padding_mask);
// Fused (1/sqrt(d)) Q K^T -> mask -> softmax -> P V for the encoder, with the
// reference's rounding points (scores and probabilities rounded to fp16).
// ctx ([B,h,S,d] fp16) and ctx_q ([B*S, h*d] int8) are both optional.
int encself_attention_f16(const __half* q, const __half* k, const __half* v, const int* pad_mask,
                          __half* ctx, int8_t* ctx_q, float quant_scale, int batch, int seq_len,
                          int head_num, int dim_per_head, hipStream_t s);
// The same attention fed by the int8 output of the QKV product ([batch * seq_len,
// 3 * hidden] codes) and the fp16 bias [3 * hidden]: each element is dequantised as
// ker_arrange_encself_qkv_i8I would have stored it, while it is staged.
int encself_attention_i8qkv(const int8_t* qkv, const __half* qkv_bias, float dequant_scale,
                            const int* pad_mask, __half* ctx, int8_t* ctx_q, float quant_scale,
                            int batch, int seq_len, int head_num, int dim_per_head, hipStream_t s);

// QKV projection + encoder attention of a (sequence, head) pair in one kernel
// (qkv_attn_kernels.hip): x int8 [batch * seq_len, hidden], qkv_weight int8 [3 * hidden, hidden],
// ctx_q int8 [batch * seq_len, hidden]; byte-identical to gemm_i8_i8o (alpha = requant_alpha)
// followed by encself_attention_i8qkv.  Needs dim_per_head 64, seq_len <= 128, hidden % 128 == 0.
bool qkv_attention_fused_supported(int batch, int seq_len, int head_num, int dim_per_head);
void qkv_attention_time_next_launch(hipEvent_t start, hipEvent_t stop);
int qkv_attention_i8(const int8_t* x, const int8_t* qkv_weight, const __half* qkv_bias,
                     const int* pad_mask, int8_t* ctx_q, float requant_alpha, float dequant_scale,
                     float quant_scale, int batch, int seq_len, int head_num, int dim_per_head,
                     hipStream_t s, const int* plan = nullptr);
// The plan of such launches (batch * head_num ints, made once per padding mask): workgroups take
// their (sequence, head) pairs longest sequence first, paired on a compute unit with the
// shortest, and leave out the 32-token blocks that hold nothing but padding.  Same bytes on
// the rows of tokens that are not padding, zeros on the others.
bool qkv_attention_plan_supported(int batch, int seq_len, int head_num);
bool qkv_attention_plan_enable(bool on);  // what the models do (default on); returns the previous setting
bool qkv_attention_plan_enabled();
int qkv_attention_plan(const int* pad_mask, int* plan, int batch, int seq_len, int head_num,
                       hipStream_t s);

// ---- int8 MFMA GEMM (gemm_i8.hip) -----------------------------------------------------
// C[M,N] = A[M,K] * W[N,K]^T, both operands K-contiguous.
int gemm_i8_i32o(const int8_t* A, const int8_t* W, int32_t* C, int M, int N, int K,
                 hipStream_t s);
// K split into `ksplit` ranges; range p writes the plane C + p * M * N.  Returns the ksplit
// actually used (1 when the shape does not split evenly) in *used.
int gemm_i8_i32o_splitk(const int8_t* A, const int8_t* W, int32_t* C, int M, int N, int K,
                        int ksplit, int* used, hipStream_t s);
// The split the library prefers for an int32-output GEMM of this shape (1 = none).
int gemm_i8_preferred_ksplit(int M, int N, int K);
int gemm_i8_i8o(const int8_t* A, const int8_t* W, int8_t* C, int M, int N, int K, float alpha,
                hipStream_t s);
// Fused epilogues (fp16 models).  Each produces exactly the bits of the int8-output GEMM
// followed by the stand-alone kernel it absorbs.
//   act: ActKind (0 GELU, 1 ReLU, 2 ReLU with the narrow unsigned clip)
int gemm_i8_bias_act_i8o(const int8_t* A, const int8_t* W, int8_t* C, const __half* bias, int M,
                         int N, int K, float alpha, float dequant_scale, float quant_scale,
                         float clip_max, int act, hipStream_t s);
// The same epilogue as a table lookup: `lut` [N, 256] int8, entry [n][code + 128] = what
// gemm_i8_bias_act_i8o produces for requantised code `code` in column n; built once per
// weight matrix by build_act_lut.  Bit-identical to gemm_i8_bias_act_i8o.
int build_act_lut(int8_t* lut, const __half* bias, int N, float dequant_scale, float quant_scale,
                  float clip_max, int act, hipStream_t s);
// Decode-step QKV product with ker_arrange_decself_qkv_i8I_i8O as its epilogue: q codes to
// new_q [M, hidden], k and v codes to slot step_id of the caches [M, heads, max_step, d].
int gemm_i8_decself_qkv_i8o(const int8_t* A, const int8_t* W, const __half* qkv_bias, int8_t* new_q,
                            int8_t* new_k, int8_t* new_v, int step_token_num, int hidden, int K,
                            int head_num, int max_step, int step_id, float alpha,
                            float dequant_scale, float quant_scale, hipStream_t s);
// gemm_i8_decself_qkv_i8o followed by decself_attention_i8 (step_num = step_id + 1) in one
// launch, for heads of 64 dimensions (dec_qkv_attn_kernels.hip).  ctx must not alias x.
bool decself_qkv_attention_supported(int rows, int hidden, int head_num, int max_step);
bool decself_qkv_attention_enable(bool on);  // what the models do; returns the previous setting
bool decself_qkv_attention_enabled();
int decself_qkv_attention_i8(const int8_t* x, const int8_t* qkv_weight, const __half* qkv_bias,
                             int8_t* new_q, int8_t* k_cache, int8_t* v_cache, int8_t* ctx,
                             int rows, int hidden, int head_num, int max_step, int step_id,
                             float alpha, float dequant_scale, float cache_quant_scale,
                             float attn_scale, float cache_dequant_scale, float ctx_quant_scale,
                             hipStream_t s);
// Decode-step cross-attention query product with ker_arrange_encdec_q_i8I as its epilogue:
// fp16 q [batch, heads, beam, d].
int gemm_i8_encdec_q_f16(const int8_t* A, const int8_t* W, const __half* q_bias, __half* new_q,
                         int step_token_num, int hidden, int K, int beam_size, int head_num,
                         float alpha, float dequant_scale, hipStream_t s);
int gemm_i8_lut_i8o(const int8_t* A, const int8_t* W, int8_t* C, const int8_t* lut, int M, int N,
                    int K, float alpha, hipStream_t s);
//   writes q, k, v as fp16 [B, h, S, d] at new_qkv + {0, 1, 2} * max_batch_dim
int gemm_i8_qkv_arrange_f16(const int8_t* A, const int8_t* W, __half* new_qkv,
                            const __half* qkv_bias, long max_batch_dim, int batch_tokens,
                            int hidden, int K, int seq_len, int head_num, float alpha,
                            float dequant_scale, hipStream_t s);
// Name of the kernel instantiation the dispatcher picks for a shape (for profiles);
// epilogue is "EpiI8", "EpiI32", "EpiGeluI8", "EpiReluI8" or "EpiQkvF16".
std::string gemm_i8_kernel_name(int M, int N, int K, const char* epilogue);
const char* gemm_i8_act_epilogue_name(int act);
// The next int8 GEMM launched from this thread records kernel-exact begin / end
// timestamps into the two events (hipExtLaunchKernelGGL), then the hook clears itself.
void gemm_i8_time_next_launch(hipEvent_t start, hipEvent_t stop);
// Counts the changes of the process-wide route switches below (tile kernel, decode-step
// kernel, fused decode attention, activation table kernel).  Whoever keeps launches recorded
// (the models' step graphs) compares it with the value it recorded under and drops what it
// holds when a switch has moved since.
unsigned long route_epoch();
void route_epoch_bump();
// A/B switch: route large products to the persistent kernels instead of the one-tile-per-
// workgroup kernel (on by default)
bool gemm_i8_enable_tile_kernel(bool on);  // returns the previous setting
// The same for the decode-step products (M <= 64): the 16 x 16 x 64 kernel (default, where a
// workgroup's K range is a multiple of 256) or the 32 x 32 x 32 one; same bits.
bool gemm_i8_enable_skinny16_kernel(bool on);
bool bias_act_enable_lut_kernel(bool on);  // returns the previous setting
// register-resident int8 MFMA loop (measurement aid): out needs workgroups * 256 ints; *ops
// receives the integer operations of one launch
int mfma_i8_peak_probe(int* out, int workgroups, int iters, double* ops, hipStream_t s);

// ---- feed-forward segment of an encoder layer in one launch (xcd_ffn_kernels.hip) ----------
// FFN1 with the tabulated epilogue -> FFN2 -> dequantise + residual (+ colsum) + layer norm
// (+ quantise), the rows dealt to the 8 XCDs whose workgroups synchronise through their L2.
// Same bytes as gemm_i8_lut_i8o + gemm_i8_i32o + residual_bias_ln_i8O / residual_bias_ln_i32I.
bool ffn_segment_supported(int M, int H, int I);
size_t ffn_segment_sync_words();  // unsigned words of device memory behind `sync`
int ffn_segment_i8(const int8_t* x, const int8_t* w1, const int8_t* lut1, float alpha1, int8_t* act,
                   const int8_t* w2, int32_t* acc, __half* residual, __half* out_t, int8_t* out_q,
                   const __half* scale, const __half* bias, const __half* residual_bias,
                   const __half* colsum, int M, int H, int I, float dequant_scale,
                   float quant_scale, bool is_post_ln, bool final_ln, unsigned* sync,
                   unsigned* launches, int spin_limit, hipStream_t s);
void ffn_segment_time_next_launch(hipEvent_t start, hipEvent_t stop);
void ffn_segment_stamps(unsigned long long* dev);  // 256 x 8 clock values per launch, or null
// what the models do (off by default: measured no faster than the three launches; returns the
// previous setting), and the process-wide
// claim that keeps two models from running the segment kernel at the same time
bool ffn_segment_enable(bool on);
bool ffn_segment_enabled();
bool ffn_segment_claim(const void* who);
void ffn_segment_release(const void* who);

// ---- fp16 MFMA GEMM (gemm_f16.hip) ------------------------------------------------------
int gemm_f16_nt(const __half* A, const __half* W, __half* C, int M, int N, int K, hipStream_t s);
// StridedBatchGemm<T>::Forward (ops/includes/strided_batch_gemm.h:45-57); op: 0 = N, 1 = T
template <typename T>
int strided_batch_gemm(int bsz, int m, int n, int k, float alpha, float beta, int op_a, int op_b,
                       const T* A, const T* B, T* C, hipStream_t s);

// ---- decoder step (dec_kernels.hip) -----------------------------------------------------
template <typename T>
int dec_emb_i8I(const int8_t* token_emb, const T* pos_emb, const int* tokens, T* output,
                int batch_size, int beam_size, int hidden_dim, int vocab_size, int step,
                int max_step, hipStream_t s, float dequant_scale, bool scaled, bool vocab_major);
template <typename T>
int arrange_decself_qkv_i8I_i8O(int step_token_num, int hidden_size, hipStream_t s,
                                const int8_t* ori_qkv, const T* qkv_bias, int8_t* new_q,
                                int8_t* new_k, int8_t* new_v, int head_num, int dim_per_head,
                                int max_step, int step_id, float dequant_scale,
                                float quant_scale);
int decself_scores_i8(const int8_t* q, const int8_t* k_cache, int32_t* scores, int batch_head_num,
                      int step_num, int max_step, int dim_per_head, hipStream_t s);
int fuse_softmax_new_value_i32I_i8O(const int32_t* correlation, const int8_t* v, int8_t* new_v,
                                    int batch_head_num, int step_num, int max_step, int head_num,
                                    int dim_per_head, float attn_scale, float dequant_scale,
                                    float quant_scale, hipStream_t s);
int decself_attention_i8(const int8_t* q, const int8_t* k_cache, const int8_t* v_cache,
                         int8_t* new_v, int batch_head_num, int step_num, int max_step,
                         int head_num, int dim_per_head, float attn_scale, float dequant_scale,
                         float quant_scale, hipStream_t s);
template <typename T>
int arrange_encdec_q_i8I(int step_token_num, int hidden_size, hipStream_t s, const int8_t* ori_q,
                         const T* q_bias, T* new_q, int beam_size, int dim_per_head, int head_num,
                         float dequant_scale);
template <typename T>
int arrange_encdec_kv(int batch_token_num, int dec_layer_num, int hidden_size, hipStream_t s,
                      const T* ori_kv, const T* kv_bias, T* new_k, T* new_v,
                      long offset_per_layer, int batch_seq_len, int dim_per_head, int head_num);
template <typename T>
int correlation_softmax_encdec(int batch_size, int head_num_per_seq, int batch_seq_len,
                               hipStream_t s, T* correlation, const int* src_padding_mask);
int encdec_attention_f16(const __half* q, const __half* k, const __half* v, const int* pad_mask,
                         __half* ctx, int8_t* ctx_q, float quant_scale, int batch_size,
                         int beam_size, int head_num, int batch_seq_len, int dim_per_head,
                         hipStream_t s);
bool encdec_q_attention_supported(int beam_size, int head_num, int hidden, int batch_seq_len);
int encdec_q_attention_f16(const int8_t* x, const int8_t* q_weight, const __half* q_bias,
                           const __half* k, const __half* v, const int* pad_mask, int8_t* ctx_q,
                           float quant_scale, int batch_size, int beam_size, int head_num,
                           int batch_seq_len, int hidden, float alpha, float dequant_scale,
                           hipStream_t s);

// ---- beam search (beam_kernels.hip) -------------------------------------------------------
template <typename T>
int select_beam_rough_topk_i8I(const int8_t* logits, const T* logit_bias, const float* seq_probs,
                               const float* seq_score, const int* alive_seq, float dequant_scale,
                               int* can_idx, float* can_score, int* num_beam_can, int vocab_size,
                               int max_step, float length_norm, int cur_step, int step_token_num,
                               int max_thread_per_block, hipStream_t s, int beam_size,
                               float diverse_lambda, int end_id);
int refresh_result(const int* can_idx, const float* can_score, const int* num_can_per_beam,
                   const int* old_alive_seq, int* new_alive_seq, float* seq_probs,
                   float* seq_score, int* num_finish_beam, int vocab_size, int cur_step,
                   float length_norm, float diverse_lambda, int end_id, int batch_size,
                   int beam_size, int max_step, hipStream_t s);
int refresh_cache_i8(int n_layer, int rows_x2, hipStream_t s, const int* num_can_per_beam,
                     const int* can_idx, const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                     int8_t* v_new, long layer_offset, int beam_size, int dim_per_head,
                     int head_num, int vocab_size, int cur_step, int max_step, bool diverse,
                     int end_id);
int refresh_cache_by_parent_i8(int n_layer, int rows, hipStream_t s, const int* parent,
                               const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                               int8_t* v_new, long layer_offset, int beam_size, int dim_per_head,
                               int head_num, int cur_step, int max_step);
int write_trg_tokenid_pos_penalty(const int* alive_seq, float* seq_score, int* output,
                                  int max_step, int beam_size, int batch_size, int out_len,
                                  hipStream_t s);
int write_trg_tokenid_neg_penalty(const int* alive_seq, const float* seq_score, int* output,
                                  int max_step, int beam_size, int vocab_size, int end_id,
                                  int batch_size, int out_len, hipStream_t s);
int write_topk_result(const int* alive_seq, float* seq_score, int* res_seq, int vocab_size,
                      int max_step, int beam_size, int end_id, int rows, int out_len,
                      hipStream_t s);
template <typename T>
int beam_search_step_i8I(const int8_t* logits, const T* logit_bias, float* seq_probs,
                         float* seq_score, const int* old_alive_seq, int* new_alive_seq,
                         float* top_score, int* top_idx, int* parent, int* num_finished,
                         float dequant_scale, int vocab_size, int max_step, float length_norm,
                         int cur_step, int batch_size, int beam_size, int end_id, hipStream_t s,
                         float* part_ws = nullptr, size_t part_ws_words = 0);
// 4-byte words of the optional workspace `part_ws` with which the per-row top-k of the step is
// dealt to several workgroups per row (0: this shape runs one workgroup per row either way)
size_t beam_search_step_workspace_words(int batch_size, int beam_size, int vocab_size);
// the same step with its proposal workspace in a static device array (allocates nothing)
int beam_search_step_noalloc_i8I_f16(const int8_t* logits, const __half* logit_bias,
                                     float* seq_probs, float* seq_score, const int* old_alive_seq,
                                     int* new_alive_seq, int* parent, int* num_finished,
                                     float dequant_scale, int vocab_size, int max_step,
                                     float length_norm, int cur_step, int batch_size, int beam_size,
                                     int end_id, hipStream_t s);
// ---- GPT path (gpt_kernels.hip, attn_kernels.hip) ------------------------------------------
// vocab_size <= 0 disables the token-id clamp, max_step <= 0 the position check
template <typename T>
int gpt_embedding_i8I(int batch_size, int batch_seq_len, int hidden_size, hipStream_t s,
                      const int8_t* token_emb, const T* pos_emb, const int* token_id, T* output,
                      int* real_seq_len, int padding_id, int pos_offset, float dequant_scale,
                      int vocab_size, int max_step, int* zero_flag = nullptr);
// zero_flag: when given, the int it points to is cleared by the same launch (a generation
// step's "unfinished" flag)
int gpt_arrange_qkv_prefill_f16(int batch_token_num, int hidden_size, hipStream_t s,
                                const int8_t* ori_qkv, const __half* qkv_bias, __half* q_codes,
                                __half* k_codes, __half* v_deq, int8_t* k_cache, int8_t* v_cache,
                                int batch_seq_len, int dim_per_head, int head_num, int max_step,
                                float dequant_scale, float quant_scale);
int gpt_prefill_attention_f16(const __half* q_codes, const __half* k_codes, const __half* v,
                              const int* real_seq_len, __half* ctx, int8_t* ctx_q,
                              float quant_scale, float dequant_scale, int batch, int seq_len,
                              int head_num, int dim_per_head, hipStream_t s);
// the prompt pass on int8 codes end to end (gpt_prefill_kernels.hip): heads of 64, at most 1024
// tokens for the attention
bool gpt_prefill_i8_supported(int seq_len, int head_num, int dim_per_head);
// what QuantGpt's prompt pass does where the shape is covered (default: on); returns the
// previous setting
bool gpt_prefill_i8_enable(bool on);
bool gpt_prefill_i8_enabled();
int gpt_arrange_qkv_prefill_i8(int batch_token_num, int hidden_size, hipStream_t s,
                               const int8_t* ori_qkv, const __half* qkv_bias, int8_t* q_codes,
                               int8_t* k_cache, int8_t* v_cache, int batch_seq_len,
                               int dim_per_head, int head_num, int max_step, float dequant_scale,
                               float quant_scale);
int gpt_prefill_attention_i8(const int8_t* q_codes, const int8_t* k_cache, const int8_t* v_cache,
                             const int* real_seq_len, int8_t* ctx_q, float quant_scale,
                             float dequant_scale, float v_quant_scale, int batch, int seq_len,
                             int head_num, int dim_per_head, int max_step, hipStream_t s);
template <typename T>
int correlation_softmax_gpt_i32I(int batch_size, int batch_seq_len, int head_num, hipStream_t s,
                                 const int32_t* correlation, T* output, const int* real_seq_len,
                                 float attn_scale, float dequant_scale);
int gpt_scores_i8(const int8_t* q, const int8_t* k, int32_t* scores, int batch_head_num,
                  int batch_seq_len, int dim_per_head, hipStream_t s);
template <typename T>
int arrange_qkv_with_cache_i8I_i8O(int batch_token_num, int hidden_size, hipStream_t s,
                                   const int8_t* ori_qkv, const T* qkv_bias, int8_t* new_q,
                                   int8_t* new_k, const int8_t* k_cache, int8_t* new_v,
                                   const int8_t* v_cache, int batch_seq_len, int dim_per_head,
                                   int head_num, float dequant_scale, float quant_scale);
// k == 1: greedy (state unused); k in {2, 4, 8, 16, 32}: random sampling with the generator
// states `state` (16 bytes per sequence, sample_state_setup)
int topk_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len, hipStream_t s,
                    const int8_t* logits, int* old_input_ids, int* new_input_ids,
                    int vocab_size, int k, int* unfinished, int eos_id, void* state,
                    float dequant_scale);
int topp_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len, hipStream_t s,
                    const int8_t* logits, int* old_input_ids, int* new_input_ids, int vocab_size,
                    float p, int* unfinished, void* state, int eos_id, float dequant_scale);
// generator states of n sequences: {seed, sequence index, draws made = 0}
int sample_state_setup(void* state, int n, unsigned long long seed, hipStream_t s);
// ker_attention_mask_weights_i32I_launcher (inference/kernels/gptKernels_int8.h:57-61)
template <typename T>
int attention_mask_weights_i32I(int batch_size, int dst_seq_len, int src_seq_len, int head_num,
                                hipStream_t s, const int32_t* correlation, T* output,
                                const int* real_seq_len, float attn_scale, float dequant_scale);
// Encoder-decoder sampling (sample_kernels.hip): ker_topk_sample_i8I_launcher /
// ker_topp_sample_i8I_launcher of inference/kernels/transformerKernels_int8.h:123-143; ids
// [rows, max_step] in place, column batch_seq_len receives the token; k == 1 needs no state.
template <typename T>
int dec_topk_sample_i8I(int batch_size, int batch_seq_len, int max_step, int logits_seq_len,
                        hipStream_t s, const int8_t* logits, const T* logit_bias, int* ids,
                        int vocab_size, int k, int* unfinished, void* state, int eos_id,
                        float dequant_scale);
template <typename T>
int dec_topp_sample_i8I(int batch_size, int batch_seq_len, int max_step, int logits_seq_len,
                        hipStream_t s, const int8_t* logits, const T* logit_bias, int* ids,
                        int vocab_size, float p, int* unfinished, void* state, int eos_id,
                        float dequant_scale);
// the model's step with random sampling (k in {2,..,32}: top-k; k == 0: top-p with p)
int gpt_sample_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size, int max_step,
                    int cur_len, int batch_size, int* unfinished, int eos_id, int k, float p,
                    float dequant_scale, void* state, hipStream_t s);
int gpt_greedy_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size, int max_step,
                    int cur_len, int batch_size, int* unfinished, int eos_id, hipStream_t s);
int ppl_i8I(int batch_size, int batch_seq_len, hipStream_t s, const int8_t* logits,
            const int* input_ids, const int* real_seq_len, float* ppl, int vocab_size,
            float dequant_scale, float* workspace = nullptr);  // workspace: batch * seq_len floats
                                                               // -> one workgroup per position

// ---- operator kernels of the csrc layer path (layer_ops.hip); clip values are device
// ---- scalars of type T, dropout ratios must be 0 -------------------------------------
template <typename T>
int opb_quantize(int8_t* q, uint8_t* cmask, float* alpha, const T* f, const T* cmax, long numel,
                 int alpha_count, int bit, hipStream_t s);
template <typename T>
int opb_fake_quantize(uint8_t* cmask, float* alpha, T* out, const T* in, const T* cmax,
                      long numel, int bit, bool symmetry, hipStream_t s);
template <typename T>
int opb_dequantize(T* f, const int8_t* q, const T* cmax, long numel, hipStream_t s);
// q_out != nullptr selects the quantising variant
template <typename T>
int opb_layer_norm(T* ln_res, int8_t* q_out, uint8_t* cmask, T* vars, T* means, const T* inp,
                   const T* gamma, const T* beta, const T* cmax_out, int rows, int hidden,
                   hipStream_t s);
template <typename T>
int opb_attn_softmax(T* vals, const T* mask, int batch, int heads, int from_len, int to_len,
                     bool mask_future, hipStream_t s);
template <typename T>
int opb_quant_bias_add_transform_20314(T* out, uint8_t* cmask, const int8_t* in, const T* bias,
                                       const T* cmax, int d0, int d1, int d2, int d3, int d4,
                                       hipStream_t s, const T* out_cmax);
// launch_bias_add_transform_20314 (transform_kernels.cu:140-235): T [d0,d1,d2,d3,d4] + bias
// [d2,d3,d4] -> [d2,d0,d3,d1,d4]
template <typename T>
int opb_bias_add_transform_20314(T* out, const T* in, const T* bias, int d0, int d1, int d2,
                                 int d3, int d4, hipStream_t s);
// launch_concat3_dim1 (general_kernels.cu:187-234): [sz0,sz1_1,sz2] ++ [sz0,sz1_2,sz2] on dim 1
template <typename T>
int opb_concat3_dim1(const T* inp1, const T* inp2, T* out, int sz0, int sz2, int sz1_1,
                     int sz1_2, hipStream_t s);
// out_q != nullptr selects the quantising variant
template <typename T>
int opb_transform4d_0213(T* out, int8_t* out_q, uint8_t* cmask, const T* vals, const T* cmax,
                         int batch, int seq, int hidden, int nhead, int tc, hipStream_t s);
template <typename T>
int opb_dropout(T* out, const T* vals, uint8_t* mask, long total, float ratio, hipStream_t s);
template <typename T>
int opb_dropout_res_bias(T* out, const T* vals, uint8_t* mask, const T* bias, const T* residual,
                         long total, int dim, float ratio, hipStream_t s);
// act: 0 gelu, 1 relu
template <typename T>
int opb_dropout_act_bias(int act, T* out, const T* vals, uint8_t* mask, const T* bias, long total,
                         int dim, float ratio, hipStream_t s);
// qout != nullptr: int8 result; else fout receives the fake-quantised T result
template <typename T>
int opb_quant_dropout_act_bias(int act, int8_t* qout, T* fout, uint8_t* cmask_out,
                               uint8_t* cmask_in, uint8_t* dropout_mask, const int8_t* qin,
                               const T* bias, const T* cmax_out, const T* cmax_in, long total,
                               int dim, float ratio, bool symmetry, hipStream_t s);
template <typename T>
int opb_quant_dropout_res_bias(T* out, uint8_t* mask, const int8_t* qvals, const T* cmax,
                               const T* bias, const T* residual, long total, int dim, float ratio,
                               hipStream_t s);
// int8 GEMM to int8 with the scale read from device memory (alpha[0])
int gemm_i8_i8o_dev_alpha(const int8_t* A, const int8_t* W, int8_t* C, int M, int N, int K,
                          const float* alpha, hipStream_t s);
int layer_attention_f16(const __half* q, const __half* k, const __half* v, const __half* add_mask,
                        __half* ctx, int batch, int seq_len, int head_num, int dim_per_head,
                        bool mask_future, hipStream_t s);
// The same with its own number of keys (cross attention, cached decoding step).
int layer_cross_attention_f16(const __half* q, const __half* k, const __half* v,
                              const __half* add_mask, __half* ctx, int batch, int seq_len,
                              int key_len, int head_num, int dim_per_head, bool mask_future,
                              hipStream_t s);

// inference/kernels/transformerKernels.h:137-140
// compute units of the current device, read once per device (gemm_i8.hip)
int cu_count();

inline float length_norm(int length, float alpha) {
  if (alpha < 0.f) return 1.f / length;
  return std::pow((5.f + length) / 6.f, -alpha);
}

}  // namespace lsh
