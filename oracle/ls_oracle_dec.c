/*
 * Decoder half of the CPU oracle -- TEST INFRASTRUCTURE ONLY (see ls_oracle.h).
 * Plain-C restatement of the reference's int8 decoder step, beam search and
 * output kernels; every function cites the reference lines it follows.
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

static const float kFloatInfNeg = -100000000.f;   /* kernels/common.h:12 */
static const float kMinLogProb = -2000.f;         /* kernels/transformerKernels.h:12 */
static const float kLogitThreshMin = -64.f;       /* kernels/transformerKernels.h:11 */
static const float kEpsilon = 0.000000000001f;    /* kernels/transformerKernels.h:13 */

/* ------------------------------------------------------------------------- */
/* embedding                                                                   */
/* ------------------------------------------------------------------------- */
void lso_dec_emb_i8I(const int8_t* token_emb, const void* pos_emb,
                     const int* tokens, void* output, int rows, int hidden,
                     int vocab, int step, int max_step, float dequant_scale,
                     int scaled, int vocab_major, int f16) {
  float scale = dequant_scale;
  if (scaled) scale *= sqrtf((float)hidden); /* embKernels_int8.cc.cu:174-175 */
  for (int r = 0; r < rows; ++r) {
    int token = tokens[(long)r * max_step + step];
    for (int i = 0; i < hidden; ++i) {
      int8_t e = vocab_major ? token_emb[(long)token * hidden + i]
                             : token_emb[(long)i * vocab + token];
      float v = (float)e * scale + ldT(pos_emb, (long)step * hidden + i, f16);
      stT(output, (long)r * hidden + i, v, f16);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* self attention                                                              */
/* ------------------------------------------------------------------------- */
void lso_arrange_decself_qkv_i8I_i8O(const int8_t* ori_qkv, const void* qkv_bias,
                                     int8_t* new_q, int8_t* k_cache,
                                     int8_t* v_cache, int rows, int head_num,
                                     int dim_per_head, int max_step, int step_id,
                                     float dequant_scale, float quant_scale,
                                     int f16) {
  const int H = head_num * dim_per_head;
  for (int r = 0; r < rows; ++r)
    for (int part = 0; part < 3; ++part)
      for (int i = 0; i < H; ++i) {
        /* (:1410-1412, :1451-1453) the bias is added in float for both T */
        float val = (float)ori_qkv[((long)r * 3 + part) * H + i] * dequant_scale +
                    ldT(qkv_bias, (long)part * H + i, f16);
        int8_t q = lso_float2int8(val, quant_scale);
        if (part == 0) {
          new_q[(long)r * H + i] = q;
        } else {
          int head = i / dim_per_head, dim = i % dim_per_head;
          long t = (((long)r * head_num + head) * max_step + step_id) * dim_per_head + dim;
          (part == 1 ? k_cache : v_cache)[t] = q;
        }
      }
}

void lso_decself_scores(const int8_t* q, const int8_t* k_cache, int32_t* scores,
                        int rows, int head_num, int dim_per_head, int max_step,
                        int step_num) {
  for (long bh = 0; bh < (long)rows * head_num; ++bh)
    for (int j = 0; j < step_num; ++j) {
      const int8_t* qp = q + bh * dim_per_head;
      const int8_t* kp = k_cache + (bh * max_step + j) * dim_per_head;
      int32_t s = 0;
      for (int d = 0; d < dim_per_head; ++d) s += (int32_t)qp[d] * (int32_t)kp[d];
      scores[bh * max_step + j] = s;
    }
}

void lso_fuse_softmax_new_value_i32I_i8O(const int32_t* logits, const int8_t* v,
                                         int8_t* new_v, int batch_head_num,
                                         int step_num, int max_step, int head_num,
                                         int dim_per_head, float attn_scale,
                                         float dequant_scale, float quant_scale) {
  float* probs = (float*)malloc(sizeof(float) * (size_t)step_num);
  for (long bh = 0; bh < batch_head_num; ++bh) {
    float mx = kFloatInfNeg;
    for (int j = 0; j < step_num; ++j) { /* (:1530-1533) */
      float val = (float)logits[bh * max_step + j] * dequant_scale * dequant_scale * attn_scale;
      probs[j] = val;
      mx = fmaxf(mx, val);
    }
    double sum = 0.0;
    for (int j = 0; j < step_num; ++j) {
      probs[j] = expf(probs[j] - mx);
      sum += (double)probs[j];
    }
    float fsum = (float)sum;
    for (int j = 0; j < step_num; ++j) probs[j] = probs[j] / fsum; /* (:1549) */
    long row = bh / head_num, head = bh % head_num;
    for (int d = 0; d < dim_per_head; ++d) {
      double acc = 0.0; /* (:1552-1562) float atomics in the reference */
      for (int j = 0; j < step_num; ++j)
        acc += (double)((float)v[(bh * max_step + j) * dim_per_head + d] * probs[j] *
                        dequant_scale);
      new_v[row * ((long)head_num * dim_per_head) + head * dim_per_head + d] =
          lso_float2int8((float)acc, quant_scale);
    }
  }
  free(probs);
}

/* ------------------------------------------------------------------------- */
/* encoder-decoder attention                                                   */
/* ------------------------------------------------------------------------- */
void lso_arrange_encdec_q_i8I(const int8_t* ori_q, const void* q_bias, void* new_q,
                              int rows, int beam_size, int dim_per_head,
                              int head_num, float dequant_scale, int f16) {
  const int H = head_num * dim_per_head;
  for (int r = 0; r < rows; ++r) {
    int batch_id = r / beam_size, beam_id = r % beam_size;
    for (int i = 0; i < H; ++i) {
      float val;
      if (f16) /* (:1641-1645) half(code*dq) + bias as a half add */
        val = rndT((float)ori_q[(long)r * H + i] * dequant_scale, 1) + ldT(q_bias, i, 1);
      else
        val = (float)ori_q[(long)r * H + i] * dequant_scale + ldT(q_bias, i, 0);
      int head = i / dim_per_head, dim = i % dim_per_head;
      long t = (((long)batch_id * head_num + head) * beam_size + beam_id) * dim_per_head + dim;
      stT(new_q, t, val, f16);
    }
  }
}

void lso_arrange_encdec_kv(const void* ori_kv, const void* kv_bias, void* new_k,
                           void* new_v, long offset_per_layer, int batch,
                           int seq_len, int n_layer, int dim_per_head,
                           int head_num, int f16) {
  const int H = head_num * dim_per_head;
  for (long tok = 0; tok < (long)batch * seq_len; ++tok)
    for (int y = 0; y < n_layer * 2; ++y)
      for (int i = 0; i < H; ++i) {
        float val = ldT(ori_kv, (tok * n_layer * 2 + y) * H + i, f16) +
                    ldT(kv_bias, (long)y * H + i, f16); /* T add, rounded by stT */
        long seq_id = tok / seq_len, token_id = tok % seq_len;
        int head = i / dim_per_head, dim = i % dim_per_head;
        long t = ((seq_id * head_num + head) * seq_len + token_id) * dim_per_head + dim +
                 (long)(y >> 1) * offset_per_layer;
        stT((y & 1) ? new_v : new_k, t, val, f16);
      }
}

void lso_correlation_softmax_encdec(void* correlation, const int* pad_mask,
                                    int batch, int heads_x_beams, int seq_len,
                                    int f16) {
  float* e = (float*)malloc(sizeof(float) * (size_t)seq_len);
  for (int b = 0; b < batch; ++b)
    for (int y = 0; y < heads_x_beams; ++y) {
      long base = ((long)b * heads_x_beams + y) * seq_len;
      const int* mask = pad_mask + (long)b * seq_len;
      float mx = kFloatInfNeg;
      for (int j = 0; j < seq_len; ++j)
        if (!mask[j]) mx = fmaxf(mx, ldT(correlation, base + j, f16));
      double sum = 0.0;
      for (int j = 0; j < seq_len; ++j) {
        e[j] = mask[j] ? 0.f : expf(ldT(correlation, base + j, f16) - mx);
        sum += (double)e[j];
      }
      float fsum = (float)sum;
      for (int j = 0; j < seq_len; ++j) stT(correlation, base + j, e[j] / fsum, f16);
    }
  free(e);
}

void lso_attn_scores_rect(const void* q, const void* k, void* scores,
                          int batch_heads, int n_q, int n_k, int dim_per_head,
                          float alpha, int f16) {
  float a = rndT(alpha, f16);
  for (long bh = 0; bh < batch_heads; ++bh)
    for (int i = 0; i < n_q; ++i)
      for (int j = 0; j < n_k; ++j) {
        double acc = 0.0;
        for (int d = 0; d < dim_per_head; ++d)
          acc += (double)ldT(q, (bh * n_q + i) * dim_per_head + d, f16) *
                 (double)ldT(k, (bh * n_k + j) * dim_per_head + d, f16);
        stT(scores, (bh * n_q + i) * n_k + j, a * (float)acc, f16);
      }
}

void lso_attn_context_rect(const void* probs, const void* v, void* ctx,
                           int batch_heads, int n_q, int n_k, int dim_per_head,
                           int f16) {
  for (long bh = 0; bh < batch_heads; ++bh)
    for (int i = 0; i < n_q; ++i)
      for (int d = 0; d < dim_per_head; ++d) {
        double acc = 0.0;
        for (int j = 0; j < n_k; ++j)
          acc += (double)ldT(probs, (bh * n_q + i) * n_k + j, f16) *
                 (double)ldT(v, (bh * n_k + j) * dim_per_head + d, f16);
        stT(ctx, (bh * n_q + i) * dim_per_head + d, (float)acc, f16);
      }
}

void lso_gemm_T(const void* A, const void* B, void* C, int M, int N, int K, int f16) {
  /* convert once so the inner loop is plain float */
  float* a = (float*)malloc(sizeof(float) * (size_t)M * K);
  float* b = (float*)malloc(sizeof(float) * (size_t)K * N);
  for (long i = 0; i < (long)M * K; ++i) a[i] = ldT(A, i, f16);
  for (long i = 0; i < (long)K * N; ++i) b[i] = ldT(B, i, f16);
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    double* acc = (double*)calloc((size_t)N, sizeof(double));
    for (int k = 0; k < K; ++k) {
      double av = (double)a[(long)m * K + k];
      const float* br = b + (long)k * N;
      for (int n = 0; n < N; ++n) acc[n] += av * (double)br[n];
    }
    for (int n = 0; n < N; ++n) stT(C, (long)m * N + n, (float)acc[n], f16);
    free(acc);
  }
  free(a);
  free(b);
}

/* ------------------------------------------------------------------------- */
/* beam search                                                                 */
/* ------------------------------------------------------------------------- */
float lso_length_norm(int length, float alpha) {
  if (alpha < 0.f) return 1.f / (float)length;
  return powf((5.f + (float)length) / 6.f, -alpha);
}

/* kernels/common.h:118-137 as it acts on the per-thread maxima of a block of
 * `threads` threads (thread t sees the vocabulary ids congruent to t): warp
 * maxima, absent warps read as 0, max over lanes that agree modulo K, then min
 * over the K classes. */
static float rough_topk_threshold(const float* thread_max, int threads, int K) {
  float g[32];
  int warps = threads >> 5;
  for (int w = 0; w < 32; ++w) {
    if (w < warps) {
      float m = thread_max[w * 32];
      for (int l = 1; l < 32; ++l) m = fmaxf(m, thread_max[w * 32 + l]);
      g[w] = m;
    } else {
      g[w] = 0.f;
    }
  }
  float best = 0.f;
  for (int r = 0; r < K; ++r) {
    float m = g[r];
    for (int j = r + K; j < 32; j += K) m = fmaxf(m, g[j]);
    best = r == 0 ? m : fminf(best, m);
  }
  return best;
}

int lso_select_beam_rough_topk_i8I(const int8_t* logits, const void* logit_bias,
                                   const float* seq_probs, const float* seq_score,
                                   const int* alive_seq, float dequant_scale,
                                   int* can_idx, float* can_score,
                                   int* num_beam_can, int vocab_size, int max_step,
                                   float length_norm, int cur_step,
                                   int step_token_num, int max_thread_per_block,
                                   int beam_size, int end_id, int f16) {
  int total = 0;
  const int T = max_thread_per_block;
  float* tmax = (float*)malloc(sizeof(float) * (size_t)T);
  float* lgts = (float*)malloc(sizeof(float) * (size_t)vocab_size);
  for (int row = 0; row < step_token_num; ++row) {
    if (cur_step != 0 && alive_seq[(long)row * max_step + cur_step] == end_id) {
      /* finished beam: one EOS candidate carrying its score (:1697-1713) */
      num_beam_can[row + 1] = 1;
      can_score[total] = seq_score[row];
      can_idx[total] = end_id + (row % beam_size) * vocab_size;
      ++total;
      continue;
    }
    const int8_t* lr = logits + (long)row * vocab_size;
    for (int t = 0; t < T; ++t) tmax[t] = kFloatInfNeg;
    float mx = kFloatInfNeg;
    for (int v = 0; v < vocab_size; ++v) {
      float lgt = (float)lr[v] * dequant_scale + ldT(logit_bias, v, f16);
      lgts[v] = lgt;
      tmax[v % T] = fmaxf(tmax[v % T], lgt);
      mx = fmaxf(mx, lgt);
    }
    double sum = 0.0;
    for (int v = 0; v < vocab_size; ++v)
      sum += (double)expf(fmaxf(lgts[v] - mx, kLogitThreshMin));
    float log_prob_base = seq_probs[row] - logf((float)sum) - mx; /* (:1769) */
    float topk = rough_topk_threshold(tmax, T, beam_size);
    int batch_id = row / beam_size;
    int n = 0;
    for (int v = 0; v < vocab_size; ++v) {
      if (lgts[v] >= topk) {
        can_score[total] = fmaxf((lgts[v] + log_prob_base) * length_norm, kMinLogProb + 1.f) +
                           (float)batch_id * kMinLogProb; /* (:1823-1825) */
        can_idx[total] = (row - batch_id * beam_size) * vocab_size + v;
        ++total;
        ++n;
      }
    }
    num_beam_can[row + 1] = n;
  }
  num_beam_can[0] = total;
  free(tmax);
  free(lgts);
  return total;
}

typedef struct {
  float score;
  int idx;
  int pos;
} cand_t;

static int cand_cmp(const void* a, const void* b) {
  const cand_t* x = (const cand_t*)a;
  const cand_t* y = (const cand_t*)b;
  if (x->score > y->score) return -1;
  if (x->score < y->score) return 1;
  return x->pos < y->pos ? -1 : (x->pos > y->pos ? 1 : 0);
}

void lso_scan_sort_candidates(int* can_idx, float* can_score, int* num_beam_can,
                              int step_token_num) {
  int total = num_beam_can[0];
  int run = 0;
  for (int i = 0; i < step_token_num; ++i) { /* exclusive scan of [1 ..] */
    int c = num_beam_can[1 + i];
    num_beam_can[1 + i] = run;
    run += c;
  }
  cand_t* c = (cand_t*)malloc(sizeof(cand_t) * (size_t)(total > 0 ? total : 1));
  for (int i = 0; i < total; ++i) {
    c[i].score = can_score[i];
    c[i].idx = can_idx[i];
    c[i].pos = i;
  }
  qsort(c, (size_t)total, sizeof(cand_t), cand_cmp);
  for (int i = 0; i < total; ++i) {
    can_score[i] = c[i].score;
    can_idx[i] = c[i].idx;
  }
  free(c);
}

void lso_refresh_result(const int* can_idx, const float* can_score,
                        const int* num_can_per_beam, const int* old_alive_seq,
                        int* new_alive_seq, float* seq_probs, float* seq_score,
                        int* num_finish_beam, int vocab_size, int cur_step,
                        float length_norm, int end_id, int batch, int beam_size,
                        int max_step) {
  for (int b = 0; b < batch; ++b)
    for (int j = 0; j < beam_size; ++j) {
      int can_pos = num_can_per_beam[b * beam_size] + j;
      int ori = can_idx[can_pos];
      int can_beam_id = ori / vocab_size, can_vocab_id = ori % vocab_size;
      for (int t = 0; t < max_step; ++t) {
        int tok;
        if (t > cur_step + 1)
          tok = end_id;
        else if (t == cur_step + 1)
          tok = can_vocab_id;
        else
          tok = old_alive_seq[((long)b * beam_size + can_beam_id) * max_step + t];
        new_alive_seq[((long)b * beam_size + j) * max_step + t] = tok;
      }
      if (can_vocab_id != end_id) {
        seq_probs[b * beam_size + j] =
            (can_score[can_pos] - (float)b * kMinLogProb) / length_norm; /* (:1434-1436) */
      } else {
        *num_finish_beam += 1;
        seq_score[b * beam_size + j] = can_score[can_pos]; /* keeps the batch offset */
      }
    }
}

void lso_refresh_cache_i8(const int* num_can_per_beam, const int* can_idx,
                          const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                          int8_t* v_new, long cache_offset, int n_layer, int batch,
                          int beam_size, int dim_per_head, int head_num,
                          int vocab_size, int cur_step, int max_step, int end_id) {
  const long beam_bytes = (long)head_num * dim_per_head * max_step;
  for (int l = 0; l < n_layer; ++l)
    for (int b = 0; b < batch; ++b)
      for (int j = 0; j < beam_size; ++j) {
        int can_pos = num_can_per_beam[b * beam_size] + j;
        int src = can_idx[can_pos] / vocab_size;
        if (can_idx[can_pos] % vocab_size == end_id) continue; /* (:1596-1598) */
        long o = (long)l * cache_offset + ((long)b * beam_size + src) * beam_bytes;
        long n = (long)l * cache_offset + ((long)b * beam_size + j) * beam_bytes;
        for (int h = 0; h < head_num; ++h)
          for (int s = 0; s <= cur_step; ++s) {
            long p = ((long)h * max_step + s) * dim_per_head;
            memcpy(k_new + n + p, k_old + o + p, (size_t)dim_per_head);
            memcpy(v_new + n + p, v_old + o + p, (size_t)dim_per_head);
          }
      }
}

void lso_write_trg_tokenid_pos_penalty(const int* alive_seq, float* seq_score,
                                       int* output, int max_step, int beam_size,
                                       int batch, int out_len) {
  for (int b = 0; b < batch; ++b) {
    for (int t = 0; t < out_len; ++t)
      output[(long)b * out_len + t] = alive_seq[(long)b * beam_size * max_step + t + 1];
  }
  /* every block reads the score of its first beam and writes slot `batch`; with
   * blocks in ascending order slot b is still untouched when block b' > b reads
   * slot b'*beam_size >= b' (:1729-1732) */
  for (int b = 0; b < batch; ++b)
    seq_score[b] = seq_score[(long)b * beam_size] - (float)b * kMinLogProb;
}

void lso_write_trg_tokenid_neg_penalty(const int* alive_seq, const float* seq_score,
                                       int* output, int max_step, int beam_size,
                                       int end_id, int batch, int out_len) {
  for (int b = 0; b < batch; ++b) {
    float best = kFloatInfNeg;
    int res = 0;
    for (int j = 0; j < beam_size; ++j) {
      int len = 0;
      for (int t = 0; t < out_len; ++t)
        len += alive_seq[((long)b * beam_size + j) * max_step + t + 1] != end_id;
      float sc = seq_score[b * beam_size + j] - (float)b * kMinLogProb;
      sc /= ((float)len + kEpsilon);
      if (sc > best) {
        best = sc;
        res = j;
      }
    }
    for (int t = 0; t < out_len; ++t)
      output[(long)b * out_len + t] = alive_seq[((long)b * beam_size + res) * max_step + t + 1];
  }
}

void lso_write_topk_result(const int* alive_seq, float* seq_score, int* res_seq,
                           int max_step, int beam_size, int end_id, int rows,
                           int out_len) {
  for (int r = 0; r < rows; ++r) {
    for (int t = 0; t < out_len; ++t)
      res_seq[(long)r * out_len + t] = alive_seq[(long)r * max_step + t + 1];
    seq_score[r] -= (float)(r / beam_size) * kMinLogProb;
    res_seq[(long)r * out_len + out_len - 1] = end_id;
  }
}

/* ------------------------------------------------------------------------- */
/* whole decoder                                                               */
/* ------------------------------------------------------------------------- */
int lso_quant_decoder(const lso_dec_weights* w, const void* enc_out,
                      const int* pad_mask, int batch, int seq_len, int is_benchmark,
                      int output_topk, int* result, int* out_len, float* scores,
                      lso_dec_trace* trace) {
  const int H = w->hidden, I = w->inner, h = w->head_num, f16 = w->f16;
  const int L = w->n_layer, V = w->vocab, beam = w->beam_size, S = seq_len;
  const int max_step = w->max_step;
  if (H % h) return 1;
  if (seq_len > max_step) return 2; /* model/quant_decoder.cc.cu:419-421 */
  if ((I & 1) || ((H / h) & 1)) return 3;
  const int d = H / h;
  const int M = batch * beam;
  const long tokens = (long)batch * S;
  const size_t tsz = f16 ? 2 : 4;
  const float Q = 127.f;
  const float attn_scale = sqrtf(1.f / (float)d);
  long wide = I > 3 * H ? I : 3 * H;

  /* ---- project the encoder output (:489-515) ---- */
  const long kv_dim = (long)H * 2 * L;
  void* kvbuf = malloc(tsz * (size_t)(tokens * kv_dim));
  const long enc_layer = tokens * H;
  void* enc_k = malloc(tsz * (size_t)(enc_layer * L));
  void* enc_v = malloc(tsz * (size_t)(enc_layer * L));
  lso_gemm_T(enc_out, w->encdec_kv_kernel, kvbuf, (int)tokens, (int)kv_dim, H, f16);
  lso_arrange_encdec_kv(kvbuf, w->encdec_kv_bias, enc_k, enc_v, enc_layer, batch, S, L, d, h,
                        f16);
  free(kvbuf);

  /* ---- state (:86-140, :431-436) ---- */
  int* alive = (int*)malloc(sizeof(int) * (size_t)M * max_step);
  int* alive_buf = (int*)malloc(sizeof(int) * (size_t)M * max_step);
  for (long i = 0; i < (long)M * max_step; ++i) alive[i] = alive_buf[i] = w->start_id;
  float* seq_probs = (float*)malloc(sizeof(float) * (size_t)M);
  float* seq_score = (float*)calloc((size_t)M, sizeof(float));
  for (int i = 0; i < M; ++i) seq_probs[i] = (i % beam == 0) ? 0.f : kMinLogProb / 2;
  float* len_norm = (float*)malloc(sizeof(float) * (size_t)max_step);
  for (int i = 0; i < max_step; ++i) /* (:64-71) */
    len_norm[i] = w->length_penalty >= 0 ? lso_length_norm(i + 1, w->length_penalty) : 1.f;

  const long cache_layer = (long)M * max_step * H;
  int8_t* k1 = (int8_t*)calloc((size_t)(cache_layer * L), 1);
  int8_t* v1 = (int8_t*)calloc((size_t)(cache_layer * L), 1);
  int8_t* k2 = (int8_t*)calloc((size_t)(cache_layer * L), 1);
  int8_t* v2 = (int8_t*)calloc((size_t)(cache_layer * L), 1);

  void* query = malloc(tsz * (size_t)M * H);    /* _p_d_cur_step_query */
  void* qbuf = malloc(tsz * (size_t)M * H);     /* _p_d_query_buf1 */
  void* corr = malloc(tsz * (size_t)batch * h * beam * (S > max_step ? S : max_step));
  int8_t* i8_in = (int8_t*)malloc((size_t)M * wide);
  long out_sz = (long)M * wide > (long)M * V ? (long)M * wide : (long)M * V;
  int8_t* i8_out = (int8_t*)malloc((size_t)out_sz);
  long i32_sz = (long)M * H > (long)M * h * max_step ? (long)M * H : (long)M * h * max_step;
  int32_t* i32_out = (int32_t*)malloc(sizeof(int32_t) * (size_t)i32_sz);
  int* can_idx = (int*)malloc(sizeof(int) * (size_t)M * V);
  float* can_score = (float*)malloc(sizeof(float) * (size_t)M * V);
  int* can_num = (int*)malloc(sizeof(int) * (size_t)(M + 1));

  int max_decode = (max_step < S + w->extra_decode_length ? max_step
                                                          : S + w->extra_decode_length) - 1;
  int cur_step;
  int early = 0, steps_run = 0;
  for (cur_step = 0; cur_step < max_decode - 1; ++cur_step) {
    /* ---- embedding (:571-580) ---- */
    lso_dec_emb_i8I(w->tok_emb_q, w->pos_emb, alive, query, M, H, V, cur_step, max_step,
                    w->emb_clip_max / Q, 1, 1, f16);
    for (int l = 0; l < L; ++l) {
      const float* c = w->clip_max + (long)l * 19;
      int8_t* kc = k1 + (long)l * cache_layer;
      int8_t* vc = v1 + (long)l * cache_layer;
      /* ---- self attention (:617-723) ---- */
      if (l == 0)
        lso_norm_layer_resual_i8O(query, i8_in, w->self_ln_scale[0], w->self_ln_bias[0],
                                  w->b_self_out[0], M, H, Q / c[6], w->is_post_ln, f16);
      lso_gemm_i8_i8(i8_in, w->w_self_qkv[l], i8_out, M, 3 * H, H, c[0] * c[6] / (c[12] * Q));
      lso_arrange_decself_qkv_i8I_i8O(i8_out, w->b_self_qkv[l], i8_in, kc, vc, M, h, d,
                                      max_step, cur_step, c[12] / Q, Q / c[18], f16);
      lso_decself_scores(i8_in, kc, i32_out, M, h, d, max_step, cur_step + 1);
      lso_fuse_softmax_new_value_i32I_i8O(i32_out, vc, i8_in, M * h, cur_step + 1, max_step, h,
                                          d, rndT(attn_scale, f16), c[18] / Q, Q / c[7]);
      lso_gemm_i8_i8(i8_in, w->w_self_out[l], i8_out, M, H, H, c[1] * c[7] / (c[13] * Q));
      lso_residual_bias_ln_i8O(i8_out, 0, w->encdec_ln_scale[l], w->encdec_ln_bias[l],
                               w->b_encdec_out[l], i8_in, query, M, H, c[13] / Q, Q / c[8],
                               w->is_post_ln, NULL, f16);
      /* ---- encoder-decoder attention (:729-812) ---- */
      lso_gemm_i8_i8(i8_in, w->w_encdec_q[l], i8_out, M, H, H, c[2] * c[8] / (c[14] * Q));
      lso_arrange_encdec_q_i8I(i8_out, w->b_encdec_q[l], qbuf, M, beam, d, h, c[14] / Q, f16);
      const void* ek = (const char*)enc_k + tsz * (size_t)(enc_layer * l);
      const void* ev = (const char*)enc_v + tsz * (size_t)(enc_layer * l);
      lso_attn_scores_rect(qbuf, ek, corr, batch * h, beam, S, d, attn_scale, f16);
      lso_correlation_softmax_encdec(corr, pad_mask, batch, h * beam, S, f16);
      lso_attn_context_rect(corr, ev, qbuf, batch * h, beam, S, d, f16);
      lso_arrange_atten_output_i8O(qbuf, i8_in, M, beam, d, h, Q / c[9], f16);
      lso_gemm_i8_i8(i8_in, w->w_encdec_out[l], i8_out, M, H, H, c[3] * c[9] / (c[15] * Q));
      lso_residual_bias_ln_i8O(i8_out, 0, w->ffn_ln_scale[l], w->ffn_ln_bias[l], w->b_ffn2[l],
                               i8_in, query, M, H, c[15] / Q, Q / c[10], w->is_post_ln, NULL,
                               f16);
      /* ---- ffn (:815-935) ---- */
      lso_gemm_i8_i8(i8_in, w->w_ffn1[l], i8_out, M, I, H, c[4] * c[10] / (c[16] * Q));
      if (w->use_gelu)
        lso_bias_gelu_i8I_i8O(i8_out, i8_in, w->b_ffn1[l], M, I, c[16] / Q, Q / c[11], f16);
      else
        lso_bias_relu_i8I_i8O(i8_out, i8_in, w->b_ffn1[l], M, I, c[16] / Q, Q / c[11], c[11], 1,
                              f16);
      lso_gemm_i8_i32(i8_in, w->w_ffn2[l], i32_out, M, H, I);
      float dq = w->use_gelu ? c[5] * c[11] / (Q * Q) : c[5] * c[11] / (2 * Q * Q);
      const void* colsum = w->ffn2_colsum ? w->ffn2_colsum[l] : NULL;
      if (l == L - 1) {
        lso_residual_bias_ln_i8O(i32_out, 1, w->out_ln_scale, w->out_ln_bias, NULL, i8_in, query,
                                 M, H, dq, Q / w->output_ln_clip_max, w->is_post_ln, colsum, f16);
      } else {
        const float* cn = w->clip_max + (long)(l + 1) * 19;
        lso_residual_bias_ln_i8O(i32_out, 1, w->self_ln_scale[l + 1], w->self_ln_bias[l + 1],
                                 w->b_self_out[l + 1], i8_in, query, M, H, dq, Q / cn[6],
                                 w->is_post_ln, colsum, f16);
      }
    }
    /* ---- logits (:527-532) ---- */
    lso_gemm_i8_i8(i8_in, w->tok_emb_q, i8_out, M, V, H,
                   w->output_ln_clip_max * w->emb_clip_max / (w->logits_clip_max * Q));
    if (trace && trace->logits_record)
      memcpy(trace->logits_record + (long)cur_step * M * V, i8_out, (size_t)M * V);
    const int8_t* lg = i8_out;
    if (trace && trace->forced_logits && cur_step < trace->forced_steps)
      lg = trace->forced_logits + (long)cur_step * M * V;
    ++steps_run;
    /* ---- beam search (:988-1075) ---- */
    lso_select_beam_rough_topk_i8I(lg, w->logit_bias, seq_probs, seq_score, alive,
                                   w->logits_clip_max / Q, can_idx, can_score, can_num, V,
                                   max_step, len_norm[cur_step], cur_step, M, 1024, beam,
                                   w->end_id, f16);
    lso_scan_sort_candidates(can_idx, can_score, can_num, M);
    int finished = 0;
    lso_refresh_result(can_idx, can_score, can_num + 1, alive, alive_buf, seq_probs, seq_score,
                       &finished, V, cur_step, len_norm[cur_step], w->end_id, batch, beam,
                       max_step);
    {
      int* t = alive;
      alive = alive_buf;
      alive_buf = t;
    }
    if (trace && trace->alive_seq_record)
      memcpy(trace->alive_seq_record + (long)cur_step * M * max_step, alive,
             sizeof(int) * (size_t)M * max_step);
    if (trace && trace->seq_probs_record)
      memcpy(trace->seq_probs_record + (long)cur_step * M, seq_probs, sizeof(float) * (size_t)M);
    if (finished == M) {
      early = 1;
      if (!is_benchmark) break;
      continue; /* run_step returns before the cache refresh (:1053-1058) */
    }
    if (cur_step > 0) {
      lso_refresh_cache_i8(can_num + 1, can_idx, k1, v1, k2, v2, cache_layer, L, batch, beam, d,
                           h, V, cur_step, max_step, w->end_id);
      int8_t* t = k1;
      k1 = k2;
      k2 = t;
      t = v1;
      v1 = v2;
      v2 = t;
    }
  }
  /* ---- output (:454-476) ---- */
  if (output_topk) {
    if (cur_step == max_decode) cur_step -= 1;
    *out_len = cur_step + 1;
    lso_write_topk_result(alive, seq_score, result, max_step, beam, w->end_id, M, cur_step + 1);
    if (scores) memcpy(scores, seq_score, sizeof(float) * (size_t)M);
    scores = NULL;
  } else if (w->length_penalty >= 0.f || cur_step == max_decode)
    lso_write_trg_tokenid_pos_penalty(alive, seq_score, result, max_step, beam, batch,
                                      cur_step + 1);
  else
    lso_write_trg_tokenid_neg_penalty(alive, seq_score, result, max_step, beam, w->end_id,
                                      batch, cur_step + 1);
  *out_len = cur_step + 1;
  if (scores) memcpy(scores, seq_score, sizeof(float) * (size_t)batch);
  if (trace) {
    trace->steps_run = steps_run;
    trace->early_stopped = early;
  }
  free(enc_k); free(enc_v); free(alive); free(alive_buf); free(seq_probs); free(seq_score);
  free(len_norm); free(k1); free(v1); free(k2); free(v2); free(query); free(qbuf); free(corr);
  free(i8_in); free(i8_out); free(i32_out); free(can_idx); free(can_score); free(can_num);
  return 0;
}
