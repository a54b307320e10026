/*
 * GPT half of the CPU oracle -- TEST INFRASTRUCTURE ONLY (see ls_oracle.h).
 * Plain-C restatement of the reference's int8 GPT path: embedding, causal int8
 * self attention (prefill and cached step), greedy sampling, perplexity.
 */
#include "ls_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline float ldT(const void* p, long i, int f16) {
  return f16 ? lso_h2f(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
static inline void stT(void* p, long i, float v, int f16) {
  if (f16)
    ((uint16_t*)p)[i] = lso_f2h(v);
  else
    ((float*)p)[i] = v;
}
static inline float rndT(float v, int f16) { return f16 ? lso_h2f(lso_f2h(v)) : v; }

static const float kFloatInfNeg = -100000000.f; /* kernels/common.h:12 */
static const float kLogitThreshMin = -64.f;     /* kernels/transformerKernels.h:11 */

void lso_gpt_embedding_i8I(const int8_t* token_emb, const void* pos_emb,
                           const int* token_id, void* output, int* real_seq_len,
                           int padding_id, int pos_offset, float dequant_scale,
                           int batch, int seq_len, int hidden, int f16) {
  for (int b = 0; b < batch; ++b)
    for (int s = 0; s < seq_len; ++s) {
      long pos = (long)b * seq_len + s;
      int tid = token_id[pos];
      if (tid == padding_id) {
        for (int i = 0; i < hidden; ++i) stT(output, pos * hidden + i, 0.f, f16);
        continue;
      }
      real_seq_len[b] += 1; /* (:34-36) atomicAdd */
      for (int i = 0; i < hidden; ++i) {
        float v = (float)token_emb[(long)tid * hidden + i] * dequant_scale +
                  ldT(pos_emb, (long)(s + pos_offset) * hidden + i, f16);
        stT(output, pos * hidden + i, v, f16);
      }
    }
}

void lso_gpt_scores_i8(const int8_t* q, const int8_t* k, int32_t* scores,
                       int batch_heads, int seq_len, int dim_per_head) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < (long)batch_heads * seq_len; ++r) {
    long bh = r / seq_len;
    for (int j = 0; j < seq_len; ++j) {
      const int8_t* qp = q + r * dim_per_head;
      const int8_t* kp = k + (bh * seq_len + j) * dim_per_head;
      int32_t s = 0;
      for (int d = 0; d < dim_per_head; ++d) s += (int32_t)qp[d] * (int32_t)kp[d];
      scores[r * seq_len + j] = s;
    }
  }
}

void lso_correlation_softmax_gpt_i32I(const int32_t* correlation, void* output,
                                      const int* real_seq_len, int batch,
                                      int seq_len, int head_num, float attn_scale,
                                      float dequant_scale, int f16) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < (long)batch * head_num * seq_len; ++r) {
    int b = (int)(r / ((long)head_num * seq_len));
    int qpos = (int)(r % seq_len);
    long base = r * seq_len;
    if (qpos >= real_seq_len[b]) {
      for (int j = 0; j < seq_len; ++j) stT(output, base + j, 0.f, f16);
      continue;
    }
    float mx = kFloatInfNeg;
    for (int j = 0; j <= qpos; ++j) { /* (:209-212) causal: keys to the left only */
      float val = (float)correlation[base + j] * attn_scale * dequant_scale * dequant_scale;
      mx = fmaxf(mx, val);
    }
    double sum = 0.0;
    for (int j = 0; j <= qpos; ++j) {
      float val = (float)correlation[base + j] * attn_scale * dequant_scale * dequant_scale;
      sum += (double)expf(val - mx);
    }
    float fsum = (float)sum;
    for (int j = 0; j < seq_len; ++j) {
      float e = 0.f;
      if (j <= qpos) {
        float val = (float)correlation[base + j] * attn_scale * dequant_scale * dequant_scale;
        e = expf(val - mx);
      }
      stT(output, base + j, e / fsum, f16);
    }
  }
}

/* ker_attention_mask_weights_i32I (inference/kernels/gptKernels_int8.cc.cu:815-843): the last
 * dst_seq_len queries over src_seq_len keys; correlation / output [batch, head_num *
 * dst_seq_len, src_seq_len].  Rows of queries at or beyond the real length stay untouched
 * (the kernel returns before its store, :820-823). */
void lso_attention_mask_weights_i32I(const int32_t* correlation, void* output,
                                     const int* real_seq_len, int batch, int dst_seq_len,
                                     int src_seq_len, int head_num, float attn_scale,
                                     float dequant_scale, int f16) {
  const long rows_per_batch = (long)head_num * dst_seq_len;
#pragma omp parallel for schedule(static)
  for (long r = 0; r < (long)batch * rows_per_batch; ++r) {
    int b = (int)(r / rows_per_batch);
    int qpos = (int)(r % dst_seq_len) + src_seq_len - dst_seq_len; /* (:819) */
    if (qpos >= real_seq_len[b]) continue;
    long base = r * src_seq_len;
    float mx = kFloatInfNeg;
    for (int j = 0; j < src_seq_len && j <= qpos; ++j) { /* (:824-827) mask = j > qpos */
      float val = (float)correlation[base + j] * attn_scale * dequant_scale * dequant_scale;
      mx = fmaxf(mx, val);
    }
    double sum = 0.0;
    for (int j = 0; j < src_seq_len && j <= qpos; ++j) {
      float val = (float)correlation[base + j] * attn_scale * dequant_scale * dequant_scale;
      sum += (double)expf(fmaxf(kLogitThreshMin, val - mx)); /* (:837) */
    }
    float fsum = (float)sum;
    for (int j = 0; j < src_seq_len; ++j) {
      float e = 0.f;
      if (j <= qpos) {
        float val = (float)correlation[base + j] * attn_scale * dequant_scale * dequant_scale;
        e = expf(fmaxf(kLogitThreshMin, val - mx));
      }
      stT(output, base + j, e / (fsum + 1e-12f), f16); /* (:843), epsilon transformerKernels.h:13 */
    }
  }
}

void lso_arrange_qkv_with_cache_i8I_i8O(const int8_t* ori_qkv, const void* qkv_bias,
                                        int8_t* new_q, int8_t* new_k,
                                        const int8_t* k_cache, int8_t* new_v,
                                        const int8_t* v_cache, int batch,
                                        int seq_len, int dim_per_head,
                                        int head_num, float dequant_scale,
                                        float quant_scale, int f16) {
  const int H = head_num * dim_per_head;
  for (int b = 0; b < batch; ++b)
    for (int h = 0; h < head_num; ++h)
      for (int t = 0; t < seq_len; ++t)
        for (int d = 0; d < dim_per_head; ++d) {
          long target = (((long)b * head_num + h) * seq_len + t) * dim_per_head + d;
          if (t < seq_len - 1) {
            long old = (((long)b * head_num + h) * (seq_len - 1) + t) * dim_per_head + d;
            new_k[target] = k_cache[old];
            new_v[target] = v_cache[old];
          } else {
            int i = h * dim_per_head + d;
            for (int part = 0; part < 3; ++part) {
              float val = (float)ori_qkv[((long)b * 3 + part) * H + i] * dequant_scale +
                          ldT(qkv_bias, (long)part * H + i, f16);
              int8_t q = lso_float2int8(val, quant_scale);
              if (part == 0)
                new_q[((long)b * head_num + h) * dim_per_head + d] = q;
              else if (part == 1)
                new_k[target] = q;
              else
                new_v[target] = q;
            }
          }
        }
}

void lso_topk_sample_i8I_greedy(const int8_t* logits, int* old_input_ids,
                                int* new_input_ids, int vocab_size, int batch,
                                int seq_len, int logits_seq_len, int* unfinished,
                                int eos_id, float dequant_scale) {
  for (int b = 0; b < batch; ++b) {
    for (int t = 0; t < seq_len; ++t)
      new_input_ids[(long)b * (seq_len + 1) + t] = old_input_ids[(long)b * seq_len + t];
    int tok;
    if (old_input_ids[(long)b * seq_len + seq_len - 1] == eos_id) {
      tok = eos_id; /* (:263-277) */
    } else {
      const int8_t* lr = logits + ((long)b * logits_seq_len + logits_seq_len - 1) * vocab_size;
      float mx = kFloatInfNeg;
      for (int v = 0; v < vocab_size; ++v) mx = fmaxf(mx, (float)lr[v] * dequant_scale);
      tok = vocab_size;
      for (int v = 0; v < vocab_size; ++v)
        if ((float)lr[v] * dequant_scale == mx) {
          tok = v;
          break;
        }
      if (tok != eos_id) *unfinished = 1;
    }
    new_input_ids[(long)b * (seq_len + 1) + seq_len] = tok;
  }
  /* the sampled ids behind the old array (:458-460); done last so that the copy
   * above has read every old id first */
  for (int b = 0; b < batch; ++b)
    old_input_ids[(long)batch * seq_len + b] = new_input_ids[(long)b * (seq_len + 1) + seq_len];
}

void lso_ppl_i8I(const int8_t* logits, const int* input_ids, const int* real_seq_len,
                 float* ppl, int vocab_size, float dequant_scale, int batch,
                 int seq_len) {
  for (int b = 0; b < batch; ++b) {
    int len = real_seq_len[b];
    double acc = 0.0; /* float atomics in the reference */
    for (int s = 0; s < seq_len; ++s) {
      if (s >= len - 1) continue;
      long tok = (long)b * seq_len + s;
      const int8_t* lr = logits + tok * vocab_size;
      float mx = kFloatInfNeg;
      for (int v = 0; v < vocab_size; ++v) mx = fmaxf(mx, (float)lr[v] * dequant_scale);
      double sum = 0.0;
      for (int v = 0; v < vocab_size; ++v)
        sum += (double)expf(fmaxf((float)lr[v] * dequant_scale - mx, kLogitThreshMin));
      int target = input_ids[tok + 1];
      float log_prob = ((float)lr[target] * dequant_scale - mx - logf((float)sum)) /
                       (float)(len - 1);
      acc += (double)(-log_prob);
    }
    ppl[b] += (float)acc;
  }
}

/* ------------------------------------------------------------------------- */
/* whole model                                                                 */
/* ------------------------------------------------------------------------- */
typedef struct {
  const lso_gpt_weights* w;
  int batch;
  int8_t *k_cache, *v_cache; /* [n_layer][batch, head, max_step, d] */
  void* query;               /* residual stream [rows, H] */
  int8_t *i8_in, *i8_out;
  int32_t* i32_out;
  long cache_layer;
} gpt_state;

/* FFN block + the LayerNorm that follows it (model/quant_gpt_encoder.cc.cu:646-712) */
static void gpt_ffn(gpt_state* st, int l, int rows) {
  const lso_gpt_weights* w = st->w;
  const int H = w->hidden, I = w->inner, f16 = w->f16;
  const float Q = 127.f;
  const float* c = w->clip_max + (long)l * 12;
  lso_gemm_i8_i8(st->i8_in, w->w_ffn1[l], st->i8_out, rows, I, H, c[2] * c[6] / (c[10] * Q));
  lso_bias_gelu_i8I_i8O(st->i8_out, st->i8_in, w->b_ffn1[l], rows, I, c[10] / Q, Q / c[7], f16);
  lso_gemm_i8_i32(st->i8_in, w->w_ffn2[l], st->i32_out, rows, H, I);
  float dq = c[3] * c[7] / (Q * Q);
  if (l == w->n_layer - 1) {
    lso_residual_bias_ln_i8O(st->i32_out, 1, w->out_ln_scale, w->out_ln_bias, NULL, st->i8_in,
                             st->query, rows, H, dq, Q / w->output_ln_clip_max, 0, NULL, f16);
  } else {
    const float* cn = w->clip_max + (long)(l + 1) * 12;
    lso_residual_bias_ln_i8O(st->i32_out, 1, w->ln1_scale[l + 1], w->ln1_bias[l + 1],
                             w->b_out[l + 1], st->i8_in, st->query, rows, H, dq, Q / cn[4], 0,
                             NULL, f16);
  }
}

/* prompt pass over all positions (:470-560); leaves the LayerNorm-ed int8 hidden
 * states of the last layer in st->i8_in */
static void gpt_prefill(gpt_state* st, const int* ids, int seq_len, int* real_seq_len) {
  const lso_gpt_weights* w = st->w;
  const int H = w->hidden, h = w->head_num, d = H / h, f16 = w->f16, B = st->batch;
  const int rows = B * seq_len;
  const size_t tsz = f16 ? 2 : 4;
  const float Q = 127.f;
  const float attn_scale = rndT(sqrtf(1.f / (float)d), f16);
  lso_gpt_embedding_i8I(w->tok_emb_q, w->pos_emb, ids, st->query, real_seq_len, w->padding_id, 0,
                        w->emb_clip_max / Q, B, seq_len, H, f16);
  int8_t* q8 = (int8_t*)malloc((size_t)rows * H);
  int8_t* k8 = (int8_t*)malloc((size_t)rows * H);
  int8_t* v8 = (int8_t*)malloc((size_t)rows * H);
  void* dv = malloc(tsz * (size_t)rows * H);
  int32_t* corr = (int32_t*)malloc(sizeof(int32_t) * (size_t)B * h * seq_len * seq_len);
  void* probs = malloc(tsz * (size_t)B * h * seq_len * seq_len);
  void* ctx = malloc(tsz * (size_t)rows * H);
  for (int l = 0; l < w->n_layer; ++l) {
    const float* c = w->clip_max + (long)l * 12;
    if (l == 0)
      lso_norm_layer_resual_i8O(st->query, st->i8_in, w->ln1_scale[0], w->ln1_bias[0],
                                w->b_out[0], rows, H, Q / c[4], 0, f16);
    lso_gemm_i8_i8(st->i8_in, w->w_qkv[l], st->i8_out, rows, 3 * H, H, c[0] * c[4] / (c[8] * Q));
    lso_arrange_encself_qkv_i8I_i8O(st->i8_out, w->b_qkv[l], q8, k8, v8, dv, B, seq_len, d, h,
                                    c[8] / Q, Q / c[11], f16);
    /* keep the keys / values in the fixed-stride cache for the sampling steps */
    for (long bh = 0; bh < (long)B * h; ++bh)
      for (int s = 0; s < seq_len; ++s) {
        long dst = (long)l * st->cache_layer + (bh * w->max_step + s) * d;
        memcpy(st->k_cache + dst, k8 + (bh * seq_len + s) * d, (size_t)d);
        memcpy(st->v_cache + dst, v8 + (bh * seq_len + s) * d, (size_t)d);
      }
    lso_gpt_scores_i8(q8, k8, corr, B * h, seq_len, d);
    lso_correlation_softmax_gpt_i32I(corr, probs, real_seq_len, B, seq_len, h, attn_scale,
                                     c[11] / Q, f16);
    lso_attn_context(probs, dv, ctx, B * h, seq_len, d, f16);
    lso_arrange_atten_output_i8O(ctx, st->i8_in, rows, seq_len, d, h, Q / c[5], f16);
    lso_gemm_i8_i8(st->i8_in, w->w_out[l], st->i8_out, rows, H, H, c[1] * c[5] / (c[9] * Q));
    lso_residual_bias_ln_i8O(st->i8_out, 0, w->ln2_scale[l], w->ln2_bias[l], w->b_ffn2[l],
                             st->i8_in, st->query, rows, H, c[9] / Q, Q / c[6], 0, NULL, f16);
    gpt_ffn(st, l, rows);
  }
  free(q8); free(k8); free(v8); free(dv); free(corr); free(probs); free(ctx);
}

/* one cached step for the token at position cur_len-1 (:563-643) */
static void gpt_step(gpt_state* st, const int* last_ids, int cur_len, int* real_seq_len) {
  const lso_gpt_weights* w = st->w;
  const int H = w->hidden, h = w->head_num, d = H / h, f16 = w->f16, B = st->batch;
  const float Q = 127.f;
  const float attn_scale = rndT(sqrtf(1.f / (float)d), f16);
  lso_gpt_embedding_i8I(w->tok_emb_q, w->pos_emb, last_ids, st->query, real_seq_len,
                        w->padding_id, cur_len - 1, w->emb_clip_max / Q, B, 1, H, f16);
  for (int l = 0; l < w->n_layer; ++l) {
    const float* c = w->clip_max + (long)l * 12;
    int8_t* kc = st->k_cache + (long)l * st->cache_layer;
    int8_t* vc = st->v_cache + (long)l * st->cache_layer;
    if (l == 0)
      lso_norm_layer_resual_i8O(st->query, st->i8_in, w->ln1_scale[0], w->ln1_bias[0],
                                w->b_out[0], B, H, Q / c[4], 0, f16);
    lso_gemm_i8_i8(st->i8_in, w->w_qkv[l], st->i8_out, B, 3 * H, H, c[0] * c[4] / (c[8] * Q));
    /* same arithmetic as ker_arrange_qkv_with_cache_i8I_i8O, appending in place */
    lso_arrange_decself_qkv_i8I_i8O(st->i8_out, w->b_qkv[l], st->i8_in, kc, vc, B, h, d,
                                    w->max_step, cur_len - 1, c[8] / Q, Q / c[11], f16);
    lso_decself_scores(st->i8_in, kc, st->i32_out, B, h, d, w->max_step, cur_len);
    lso_fuse_softmax_new_value_i32I_i8O(st->i32_out, vc, st->i8_in, B * h, cur_len, w->max_step,
                                        h, d, attn_scale, c[11] / Q, Q / c[5]);
    lso_gemm_i8_i8(st->i8_in, w->w_out[l], st->i8_out, B, H, H, c[1] * c[5] / (c[9] * Q));
    lso_residual_bias_ln_i8O(st->i8_out, 0, w->ln2_scale[l], w->ln2_bias[l], w->b_ffn2[l],
                             st->i8_in, st->query, B, H, c[9] / Q, Q / c[6], 0, NULL, f16);
    gpt_ffn(st, l, B);
  }
}

static int gpt_alloc(gpt_state* st, const lso_gpt_weights* w, int batch, int seq_len) {
  const int H = w->hidden, I = w->inner;
  if (H % w->head_num) return 1;
  if (seq_len > w->max_step) return 2;
  if ((I & 1) || ((H / w->head_num) & 1)) return 3;
  memset(st, 0, sizeof(*st));
  st->w = w;
  st->batch = batch;
  const long rows = (long)batch * seq_len;
  const size_t tsz = w->f16 ? 2 : 4;
  long wide = I > 3 * H ? I : 3 * H;
  st->cache_layer = (long)batch * w->max_step * H;
  st->k_cache = (int8_t*)calloc((size_t)(st->cache_layer * w->n_layer), 1);
  st->v_cache = (int8_t*)calloc((size_t)(st->cache_layer * w->n_layer), 1);
  st->query = malloc(tsz * (size_t)rows * H);
  st->i8_in = (int8_t*)malloc((size_t)rows * wide);
  st->i8_out = (int8_t*)malloc((size_t)rows * wide);
  long i32n = rows * H > (long)batch * w->head_num * w->max_step
                  ? rows * H
                  : (long)batch * w->head_num * w->max_step;
  st->i32_out = (int32_t*)malloc(sizeof(int32_t) * (size_t)i32n);
  return 0;
}

static void gpt_free(gpt_state* st) {
  free(st->k_cache); free(st->v_cache); free(st->query); free(st->i8_in); free(st->i8_out);
  free(st->i32_out);
}

int lso_quant_gpt_ppl(const lso_gpt_weights* w, const int* token_ids, int batch,
                      int seq_len, float* ppl) {
  gpt_state st;
  int rc = gpt_alloc(&st, w, batch, seq_len);
  if (rc) return rc;
  const int H = w->hidden, V = w->vocab;
  const float Q = 127.f;
  int* real_len = (int*)calloc((size_t)batch, sizeof(int));
  gpt_prefill(&st, token_ids, seq_len, real_len);
  const long rows = (long)batch * seq_len;
  int8_t* logits = (int8_t*)malloc((size_t)rows * V);
  lso_gemm_i8_i8(st.i8_in, w->tok_emb_q, logits, (int)rows, V, H,
                 w->output_ln_clip_max * w->emb_clip_max / (w->logits_clip_max * Q));
  for (int b = 0; b < batch; ++b) ppl[b] = 0.f;
  lso_ppl_i8I(logits, token_ids, real_len, ppl, V, w->logits_clip_max / Q, batch, seq_len);
  free(logits);
  free(real_len);
  gpt_free(&st);
  return 0;
}

int lso_quant_gpt_sample(const lso_gpt_weights* w, const int* token_ids, int batch,
                         int seq_len, int is_benchmark, int* out_ids, int* out_len,
                         const int8_t* forced_logits, int forced_steps,
                         int8_t* logits_record, int* steps_run) {
  gpt_state st;
  int rc = gpt_alloc(&st, w, batch, seq_len);
  if (rc) return rc;
  const int H = w->hidden, V = w->vocab, max_step = w->max_step;
  const float Q = 127.f;
  const float alpha = w->output_ln_clip_max * w->emb_clip_max / (w->logits_clip_max * Q);
  int max_seq_len = seq_len + w->extra_decode_length < max_step ? seq_len + w->extra_decode_length
                                                                : max_step;
  int* real_len = (int*)calloc((size_t)batch, sizeof(int));
  int* ids = (int*)malloc(sizeof(int) * (size_t)batch * max_step); /* [batch, max_step] */
  int* last = (int*)malloc(sizeof(int) * (size_t)batch);
  int8_t* hid = (int8_t*)malloc((size_t)batch * H);
  int8_t* logits = (int8_t*)malloc((size_t)batch * V);
  for (int b = 0; b < batch; ++b)
    memcpy(ids + (long)b * max_step, token_ids + (long)b * seq_len, sizeof(int) * (size_t)seq_len);

  int cur_len = seq_len, steps = 0;
  gpt_prefill(&st, token_ids, seq_len, real_len);
  for (int b = 0; b < batch; ++b) /* hidden states of the last position */
    memcpy(hid + (long)b * H, st.i8_in + ((long)b * seq_len + seq_len - 1) * H, (size_t)H);
  for (;;) {
    /* ---- sample one token (:399-441, :443-487) ---- */
    lso_gemm_i8_i8(hid, w->tok_emb_q, logits, batch, V, H, alpha);
    if (logits_record) memcpy(logits_record + (long)steps * batch * V, logits, (size_t)batch * V);
    const int8_t* lg = logits;
    if (forced_logits && steps < forced_steps) lg = forced_logits + (long)steps * batch * V;
    int unfinished = 0;
    for (int b = 0; b < batch; ++b) {
      int tok;
      if (ids[(long)b * max_step + cur_len - 1] == w->eos_id) {
        tok = w->eos_id;
      } else {
        const int8_t* lr = lg + (long)b * V;
        int best = 0;
        for (int v = 1; v < V; ++v)
          if (lr[v] > lr[best]) best = v; /* dequantisation is monotone; lowest id on ties */
        tok = best;
        if (tok != w->eos_id) unfinished = 1;
      }
      ids[(long)b * max_step + cur_len] = tok;
      last[b] = tok;
    }
    ++steps;
    ++cur_len;
    /* (:347-353) after the prompt pass the run ends when nothing is unfinished, benchmark
     * mode or not; (:380-381) later steps honour benchmark mode */
    if (steps == 1) {
      if (!unfinished || cur_len >= max_seq_len) break;
    } else {
      if (!unfinished && !is_benchmark) break;
      if (cur_len >= max_seq_len) break;
    }
    gpt_step(&st, last, cur_len, real_len);
    memcpy(hid, st.i8_in, (size_t)batch * H);
  }
  for (int b = 0; b < batch; ++b)
    memcpy(out_ids + (long)b * cur_len, ids + (long)b * max_step, sizeof(int) * (size_t)cur_len);
  *out_len = cur_len;
  if (steps_run) *steps_run = steps;
  free(real_len); free(ids); free(last); free(hid); free(logits);
  gpt_free(&st);
  return 0;
}
