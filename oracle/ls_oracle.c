/*
 * CPU oracle for the int8 transformer-layer forward path -- TEST INFRASTRUCTURE
 * ONLY (see ls_oracle.h).  Plain C, no dependencies beyond libm / OpenMP.
 * Build: see oracle/Makefile (-O3 -ffp-contract=off -fno-fast-math).
 */
#include "ls_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* binary16 <-> binary32                                                       */
/* ------------------------------------------------------------------------- */
float lso_h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t lso_f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u : 0));
  }
  if (ax >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* <= 2^-25 rounds to zero */
    return sign;
  }
  int e = (int)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u;
  int shift; /* bits to drop from the 24-bit significand */
  uint32_t base;
  if (e < -14) { /* subnormal half */
    shift = 13 + (-14 - e);
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  return (uint16_t)(sign | (base + q)); /* carry into exponent is correct */
}

/* T-typed load/store */
static inline float ldT(const void* p, long i, int f16) {
  return f16 ? lso_h2f(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
static inline void stT(void* p, long i, float v, int f16) {
  if (f16)
    ((uint16_t*)p)[i] = lso_f2h(v);
  else
    ((float*)p)[i] = v;
}
/* round a float to T and back */
static inline float rndT(float v, int f16) { return f16 ? lso_h2f(lso_f2h(v)) : v; }
/* kernels/common.h:217-227 safe_half_to_float: clamp to +-1e5 (f16 only) */
static inline float ldT_safe(const void* p, long i, int f16) {
  float v = ldT(p, i, f16);
  if (f16) v = fmaxf(fminf(100000.f, v), -100000.f);
  return v;
}

static const float LN_EPSILON = 1e-12f; /* kernels/transformerKernels.h:13 */

/* ------------------------------------------------------------------------- */
/* scalar quantisers                                                           */
/* ------------------------------------------------------------------------- */
int8_t lso_float2int8(float x, float quant_scale) {
  float i8_f = x * quant_scale;
  int32_t i8 = (int32_t)floorf(i8_f + 0.5f);
  i8 = i8 < -127 ? -127 : (i8 > 127 ? 127 : i8);
  return (int8_t)i8;
}

int8_t lso_posfloat2int8(float x, float quant_scale, float clip_max) {
  float i8_f = x * 2 * quant_scale - quant_scale * clip_max;
  int32_t i8 = (int32_t)floorf(i8_f + 0.5f);
  i8 = i8 < -127 ? -127 : (i8 > 127 ? 127 : i8);
  return (int8_t)i8;
}

void lso_quantize_tensor(const void* in, int8_t* out, long n, float quant_scale,
                         int f16) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; ++i) out[i] = lso_float2int8(ldT(in, i, f16), quant_scale);
}

void lso_dequantize_tensor(const int32_t* in, void* out, long n,
                           float dequant_scale, int f16) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; ++i) stT(out, i, (float)in[i] * dequant_scale, f16);
}

/* ------------------------------------------------------------------------- */
/* LayerNorm family                                                            */
/* ------------------------------------------------------------------------- */
/* two-pass mean / rstd of one row held in float */
static void row_stats(const float* row, int hidden, float* mean, float* rstd) {
  double s = 0.0;
  for (int i = 0; i < hidden; ++i) s += row[i];
  float m = (float)s / (float)hidden;
  double v = 0.0;
  for (int i = 0; i < hidden; ++i) {
    float t = row[i] - m;
    v += (double)(t * t);
  }
  *mean = m;
  *rstd = 1.0f / sqrtf((float)v / (float)hidden + LN_EPSILON);
}

void lso_norm_layer_resual_i8O(void* input, int8_t* output, const void* scale,
                               const void* bias, const void* residual_bias,
                               int tokens, int hidden, float quant_scale,
                               int is_post_ln, int f16) {
#pragma omp parallel
  {
    float* row = (float*)malloc(sizeof(float) * (size_t)hidden);
#pragma omp for schedule(static)
    for (int t = 0; t < tokens; ++t) {
      long base = (long)t * hidden;
      for (int i = 0; i < hidden; ++i) row[i] = ldT_safe(input, base + i, f16);
      float mean, rstd;
      row_stats(row, hidden, &mean, &rstd);
      for (int i = 0; i < hidden; ++i) {
        float out_f = (row[i] - mean) * rstd * ldT(scale, i, f16) + ldT(bias, i, f16);
        output[base + i] = lso_float2int8(out_f, quant_scale);
        float keep = is_post_ln ? out_f : row[i];
        /* both T variants add in float and round once (:199-203, :269-277) */
        stT(input, base + i, keep + ldT(residual_bias, i, f16), f16);
      }
    }
    free(row);
  }
}

void lso_residual_bias_ln_i8O(const void* input, int in_is_i32,
                              const void* scale, const void* bias,
                              const void* residual_bias, int8_t* output,
                              void* residual, int tokens, int hidden,
                              float dequant_scale, float quant_scale,
                              int is_post_ln, const void* colsum, int f16) {
#pragma omp parallel
  {
    float* row = (float*)malloc(sizeof(float) * (size_t)hidden);
#pragma omp for schedule(static)
    for (int t = 0; t < tokens; ++t) {
      long base = (long)t * hidden;
      for (int i = 0; i < hidden; ++i) {
        float x = in_is_i32 ? (float)((const int32_t*)input)[base + i]
                            : (float)((const int8_t*)input)[base + i];
        float r = x * dequant_scale + ldT_safe(residual, base + i, f16);
        if (colsum) r += ldT_safe(colsum, i, f16);
        row[i] = r;
      }
      float mean, rstd;
      row_stats(row, hidden, &mean, &rstd);
      for (int i = 0; i < hidden; ++i) {
        float out_f = (row[i] - mean) * rstd * ldT_safe(scale, i, f16) +
                      ldT_safe(bias, i, f16);
        output[base + i] = lso_float2int8(out_f, quant_scale);
        float rb = residual_bias ? ldT(residual_bias, i, f16) : 0.f;
        float keep = is_post_ln ? out_f : row[i];
        /* f16: T(keep) + T(bias) as a half add (:465-469, :659-663);
         * f32: plain float add (:386-390).  rndT is the identity for f32. */
        stT(residual, base + i, rndT(keep, f16) + rb, f16);
      }
    }
    free(row);
  }
}

void lso_residual_bias_ln_i32I(const int32_t* input, const void* scale,
                               const void* bias, const void* residual,
                               void* output, int tokens, int hidden,
                               float dequant_scale, const void* colsum,
                               int f16) {
#pragma omp parallel
  {
    float* row = (float*)malloc(sizeof(float) * (size_t)hidden);
#pragma omp for schedule(static)
    for (int t = 0; t < tokens; ++t) {
      long base = (long)t * hidden;
      for (int i = 0; i < hidden; ++i) {
        float r = (float)input[base + i] * dequant_scale +
                  ldT_safe(residual, base + i, f16);
        if (colsum) r += ldT_safe(colsum, i, f16);
        row[i] = r;
      }
      float mean, rstd;
      row_stats(row, hidden, &mean, &rstd);
      for (int i = 0; i < hidden; ++i) {
        float out_f = (row[i] - mean) * rstd * ldT_safe(scale, i, f16) +
                      ldT_safe(bias, i, f16);
        stT(output, base + i, out_f, f16);
      }
    }
    free(row);
  }
}

/* ------------------------------------------------------------------------- */
/* bias + activation + requant                                                 */
/* ------------------------------------------------------------------------- */
static inline float gelu_tanh(float x) { /* kernels/common.h:17-23 */
  float cdf = 0.5f * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
  return x * cdf;
}

void lso_bias_gelu_i8I_i8O(const int8_t* input, int8_t* output,
                           const void* bias, int tokens, int feature_dim,
                           float dequant_scale, float quant_scale, int f16) {
#pragma omp parallel for schedule(static)
  for (int t = 0; t < tokens; ++t) {
    long base = (long)t * feature_dim;
    for (int i = 0; i < feature_dim; ++i) {
      float f = gelu_tanh((float)input[base + i] * dequant_scale + ldT(bias, i, f16));
      output[base + i] = lso_float2int8(f, quant_scale);
    }
  }
}

void lso_bias_relu_i8I_i8O(const int8_t* input, int8_t* output,
                           const void* bias, int tokens, int feature_dim,
                           float dequant_scale, float quant_scale,
                           float clip_max, int narrow_clip, int f16) {
#pragma omp parallel for schedule(static)
  for (int t = 0; t < tokens; ++t) {
    long base = (long)t * feature_dim;
    for (int i = 0; i < feature_dim; ++i) {
      float f = fmaxf((float)input[base + i] * dequant_scale + ldT(bias, i, f16), 0.f);
      output[base + i] = narrow_clip ? lso_posfloat2int8(f, quant_scale, clip_max)
                                     : lso_float2int8(f, quant_scale);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* head split / merge                                                          */
/* ------------------------------------------------------------------------- */
void lso_arrange_encself_qkv_i8I(const int8_t* ori_qkv, const void* qkv_bias,
                                 void* new_qkv, long max_batch_dim, int batch,
                                 int seq_len, int dim_per_head, int head_num,
                                 float dequant_scale, int f16) {
  int hidden = dim_per_head * head_num;
#pragma omp parallel for schedule(static)
  for (int tok = 0; tok < batch * seq_len; ++tok) {
    int b = tok / seq_len, s = tok % seq_len;
    for (int which = 0; which < 3; ++which) {
      for (int i = 0; i < hidden; ++i) {
        int head = i / dim_per_head, dim = i % dim_per_head;
        long target = (((long)b * head_num + head) * seq_len + s) * dim_per_head + dim;
        float x = (float)ori_qkv[((long)tok * 3 + which) * hidden + i] * dequant_scale;
        float bv = ldT(qkv_bias, (long)which * hidden + i, f16);
        /* f16: T(x) + bias as a half add (:1140-1145); f32: float add */
        stT(new_qkv, max_batch_dim * which + target, rndT(x, f16) + bv, f16);
      }
    }
  }
}

void lso_arrange_encself_qkv_i8I_i8O(const int8_t* ori_qkv,
                                     const void* qkv_bias, int8_t* new_q,
                                     int8_t* new_k, int8_t* new_v, void* d_v,
                                     int batch, int seq_len, int dim_per_head,
                                     int head_num, float dequant_scale,
                                     float quant_scale, int f16) {
  int hidden = dim_per_head * head_num;
#pragma omp parallel for schedule(static)
  for (int tok = 0; tok < batch * seq_len; ++tok) {
    int b = tok / seq_len, s = tok % seq_len;
    for (int which = 0; which < 3; ++which) {
      for (int i = 0; i < hidden; ++i) {
        int head = i / dim_per_head, dim = i % dim_per_head;
        long target = (((long)b * head_num + head) * seq_len + s) * dim_per_head + dim;
        float val = (float)ori_qkv[((long)tok * 3 + which) * hidden + i] * dequant_scale +
                    ldT(qkv_bias, (long)which * hidden + i, f16);
        int8_t q = lso_float2int8(val, quant_scale);
        if (which == 0) {
          new_q[target] = q;
        } else if (which == 1) {
          new_k[target] = q;
        } else {
          new_v[target] = q;
          stT(d_v, target, (float)q / quant_scale, f16);
        }
      }
    }
  }
}

void lso_arrange_atten_output_i8O(const void* ori_q, int8_t* new_q, int tokens,
                                  int beam_size, int dim_per_head, int head_num,
                                  float quant_scale, int f16) {
  int hidden = dim_per_head * head_num;
#pragma omp parallel for schedule(static)
  for (int tok = 0; tok < tokens; ++tok) {
    int b = tok / beam_size, s = tok % beam_size;
    for (int i = 0; i < hidden; ++i) {
      int head = i / dim_per_head, dim = i % dim_per_head;
      long src = (((long)b * head_num + head) * beam_size + s) * dim_per_head + dim;
      new_q[(long)tok * hidden + i] = lso_float2int8(ldT(ori_q, src, f16), quant_scale);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* encoder attention core                                                      */
/* ------------------------------------------------------------------------- */
void lso_correlation_softmax_encself(void* correlation, const int* pad_mask,
                                     int batch, int seq_len, int head_num,
                                     int f16) {
#pragma omp parallel for schedule(static)
  for (long row = 0; row < (long)batch * head_num * seq_len; ++row) {
    int b = (int)(row / ((long)head_num * seq_len));
    int qpos = (int)(row % seq_len);
    long base = row * seq_len;
    const int* mask = pad_mask + (long)b * seq_len;
    if (mask[qpos]) { /* padded query: whole row zeroed (:1124-1129) */
      for (int j = 0; j < seq_len; ++j) stT(correlation, base + j, 0.f, f16);
      continue;
    }
    float mx = -100000000.f; /* CUDA_FLOAT_INF_NEG, kernels/common.h:12 */
    for (int j = 0; j < seq_len; ++j)
      if (!mask[j]) mx = fmaxf(mx, ldT(correlation, base + j, f16));
    double sum = 0.0;
    for (int j = 0; j < seq_len; ++j)
      if (!mask[j]) sum += (double)expf(ldT(correlation, base + j, f16) - mx);
    float fsum = (float)sum;
    for (int j = 0; j < seq_len; ++j) {
      float v = mask[j] ? 0.f : expf(ldT(correlation, base + j, f16) - mx);
      stT(correlation, base + j, v / fsum, f16);
    }
  }
}

void lso_attn_scores(const void* q, const void* k, void* scores, int batch_heads,
                     int seq_len, int dim_per_head, float alpha, int f16) {
  float a = rndT(alpha, f16);
#pragma omp parallel for schedule(static)
  for (long r = 0; r < (long)batch_heads * seq_len; ++r) {
    long bh = r / seq_len;
    const long qoff = r * dim_per_head;
    for (int j = 0; j < seq_len; ++j) {
      long koff = (bh * seq_len + j) * dim_per_head;
      double acc = 0.0;
      for (int d = 0; d < dim_per_head; ++d)
        acc += (double)ldT(q, qoff + d, f16) * (double)ldT(k, koff + d, f16);
      stT(scores, r * seq_len + j, a * (float)acc, f16);
    }
  }
}

void lso_attn_context(const void* probs, const void* v, void* ctx,
                      int batch_heads, int seq_len, int dim_per_head, int f16) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < (long)batch_heads * seq_len; ++r) {
    long bh = r / seq_len;
    for (int d = 0; d < dim_per_head; ++d) {
      double acc = 0.0;
      for (int j = 0; j < seq_len; ++j)
        acc += (double)ldT(probs, r * seq_len + j, f16) *
               (double)ldT(v, (bh * seq_len + j) * dim_per_head + d, f16);
      stT(ctx, r * dim_per_head + d, (float)acc, f16);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* int8 GEMM                                                                   */
/* ------------------------------------------------------------------------- */
static inline int32_t dot_i8(const int8_t* a, const int8_t* b, int K) {
  int32_t s = 0;
  for (int k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)b[k];
  return s;
}

void lso_gemm_i8_i32(const int8_t* A, const int8_t* W, int32_t* C, int M, int N,
                     int K) {
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    const int8_t* a = A + (long)m * K;
    for (int n = 0; n < N; ++n) C[(long)m * N + n] = dot_i8(a, W + (long)n * K, K);
  }
}

int8_t lso_requant_acc(int32_t acc, float alpha) {
  float f = (float)acc * alpha;
  int32_t q = (int32_t)floorf(f + 0.5f);
  q = q < -127 ? -127 : (q > 127 ? 127 : q);
  return (int8_t)q;
}

void lso_gemm_i8_i8(const int8_t* A, const int8_t* W, int8_t* C, int M, int N,
                    int K, float alpha) {
#pragma omp parallel for schedule(static)
  for (int m = 0; m < M; ++m) {
    const int8_t* a = A + (long)m * K;
    for (int n = 0; n < N; ++n)
      C[(long)m * N + n] = lso_requant_acc(dot_i8(a, W + (long)n * K, K), alpha);
  }
}

/* ------------------------------------------------------------------------- */
/* embedding, colsum                                                           */
/* ------------------------------------------------------------------------- */
void lso_enc_emb_i8I(const int8_t* token_emb, const void* pos_emb,
                     const int* tokens, void* output, int* pad_mask, int pad_id,
                     int batch, int seq_len, int hidden, float dequant_scale,
                     int scaled, int f16) {
  float scale = dequant_scale;
  /* (:46, :88) sqrtf of hidden re-assembled from the vector count */
  if (scaled) scale *= sqrtf((float)hidden);
#pragma omp parallel for schedule(static)
  for (int t = 0; t < batch * seq_len; ++t) {
    int s = t % seq_len;
    int token = tokens[t];
    long base = (long)t * hidden;
    if (token == pad_id) {
      pad_mask[t] = 1;
      for (int i = 0; i < hidden; ++i) stT(output, base + i, 0.f, f16);
    } else {
      pad_mask[t] = 0;
      for (int i = 0; i < hidden; ++i) {
        float v = (float)token_emb[(long)token * hidden + i] * scale +
                  ldT(pos_emb, (long)s * hidden + i, f16);
        stT(output, base + i, v, f16);
      }
    }
  }
}

void lso_scaled_colsum(const void* inp, void* out, int rows, int cols,
                       float scale, int f16) {
#pragma omp parallel for schedule(static)
  for (int c = 0; c < cols; ++c) {
    double s = 0.0;
    for (int r = 0; r < rows; ++r) s += (double)ldT(inp, (long)r * cols + c, f16);
    stT(out, c, (float)s * scale, f16);
  }
}

/* ------------------------------------------------------------------------- */
/* whole encoder stack                                                         */
/* ------------------------------------------------------------------------- */
int lso_quant_bert_encoder(const lso_bert_weights* w, const int* token_ids,
                           int batch, int seq_len, void* output, int* pad_mask,
                           const lso_bert_taps* taps) {
  const int H = w->hidden, I = w->inner, h = w->head_num, f16 = w->f16;
  if (H % h) return 1;
  if (seq_len > w->max_step) return 2;
  if ((I & 1) || ((H / h) & 1)) return 3; /* model/quant_bert_encoder.cc.cu:189-194 */
  const int d = H / h;
  const long M = (long)batch * seq_len;
  const size_t tsz = f16 ? 2 : 4;
  const float Q = 127.f;
  const int cs = w->clip_stride > 0 ? w->clip_stride : 11;
  long wide = I > 3 * H ? I : 3 * H;

  int8_t* i8_in = (int8_t*)malloc((size_t)(M * wide));
  int8_t* i8_out = (int8_t*)malloc((size_t)(M * wide));
  int32_t* i32_out = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M * H));
  void* qkv = malloc(tsz * (size_t)(3 * M * H));
  void* corr = malloc(tsz * (size_t)((long)batch * h * seq_len * seq_len));
  void* ctx = malloc(tsz * (size_t)(M * H));
  if (!i8_in || !i8_out || !i32_out || !qkv || !corr || !ctx) return 4;

  /* model/quant_bert_encoder.cc.cu:233-237 */
  lso_enc_emb_i8I(w->tok_emb_q, w->pos_emb, token_ids, output, pad_mask,
                  w->padding_id, batch, seq_len, H, w->emb_clip_max / Q, w->emb_scaled, f16);

  for (int l = 0; l < w->n_layer; ++l) {
    const float* c = w->clip_max + (long)l * cs;
    const int tap = taps && taps->tap_layer == l;
    /* ---- self attention (:271-399) ---- */
    if (l == 0) {
      lso_norm_layer_resual_i8O(output, i8_in, w->ln1_scale[0], w->ln1_bias[0],
                                w->b_out[0], (int)M, H, Q / c[4], w->is_post_ln, f16);
    }
    if (tap && taps->ln1_q) memcpy(taps->ln1_q, i8_in, (size_t)(M * H));
    lso_gemm_i8_i8(i8_in, w->w_qkv[l], i8_out, (int)M, 3 * H, H,
                   c[0] * c[4] / (c[8] * Q));
    if (tap && taps->qkv_q) memcpy(taps->qkv_q, i8_out, (size_t)(M * 3 * H));
    lso_arrange_encself_qkv_i8I(i8_out, w->b_qkv[l], qkv, M * H, batch, seq_len, d,
                                h, c[8] / Q, f16);
    const void* pq = qkv;
    const void* pk = (const char*)qkv + tsz * (size_t)(M * H);
    const void* pv = (const char*)qkv + tsz * (size_t)(2 * M * H);
    lso_attn_scores(pq, pk, corr, batch * h, seq_len, d, sqrtf(1.f / (float)d), f16);
    lso_correlation_softmax_encself(corr, pad_mask, batch, seq_len, h, f16);
    lso_attn_context(corr, pv, ctx, batch * h, seq_len, d, f16);
    if (tap && taps->ctx) memcpy(taps->ctx, ctx, tsz * (size_t)(M * H));
    lso_arrange_atten_output_i8O(ctx, i8_in, (int)M, seq_len, d, h, Q / c[5], f16);
    if (tap && taps->ctx_q) memcpy(taps->ctx_q, i8_in, (size_t)(M * H));
    lso_gemm_i8_i8(i8_in, w->w_out[l], i8_out, (int)M, H, H, c[1] * c[5] / (c[9] * Q));
    if (tap && taps->out_q) memcpy(taps->out_q, i8_out, (size_t)(M * H));
    lso_residual_bias_ln_i8O(i8_out, 0, w->ln2_scale[l], w->ln2_bias[l], w->b_ffn2[l],
                             i8_in, output, (int)M, H, c[9] / Q, Q / c[6],
                             w->is_post_ln, NULL, f16);
    if (tap && taps->ln2_q) memcpy(taps->ln2_q, i8_in, (size_t)(M * H));
    /* ---- ffn (:402-520) ---- */
    lso_gemm_i8_i8(i8_in, w->w_ffn1[l], i8_out, (int)M, I, H, c[2] * c[6] / (c[10] * Q));
    if (tap && taps->ffn1_q) memcpy(taps->ffn1_q, i8_out, (size_t)(M * I));
    if (w->use_gelu)
      lso_bias_gelu_i8I_i8O(i8_out, i8_in, w->b_ffn1[l], (int)M, I, c[10] / Q, Q / c[7], f16);
    else
      lso_bias_relu_i8I_i8O(i8_out, i8_in, w->b_ffn1[l], (int)M, I, c[10] / Q, Q / c[7],
                            c[7], 1, f16);
    if (tap && taps->act_q) memcpy(taps->act_q, i8_in, (size_t)(M * I));
    lso_gemm_i8_i32(i8_in, w->w_ffn2[l], i32_out, (int)M, H, I);
    if (tap && taps->ffn2_acc) memcpy(taps->ffn2_acc, i32_out, sizeof(int32_t) * (size_t)(M * H));
    float dq = w->use_gelu ? c[3] * c[7] / (Q * Q) : c[3] * c[7] / (2 * Q * Q);
    const void* colsum = w->ffn2_colsum ? w->ffn2_colsum[l] : NULL;
    if (l == w->n_layer - 1) {
      lso_residual_bias_ln_i32I(i32_out, w->final_ln_scale, w->final_ln_bias, output,
                                output, (int)M, H, dq, colsum, f16);
    } else {
      const float* cn = w->clip_max + (long)(l + 1) * cs;
      lso_residual_bias_ln_i8O(i32_out, 1, w->ln1_scale[l + 1], w->ln1_bias[l + 1],
                               w->b_out[l + 1], i8_in, output, (int)M, H, dq,
                               Q / cn[4], w->is_post_ln, colsum, f16);
    }
  }
  free(i8_in);
  free(i8_out);
  free(i32_out);
  free(qkv);
  free(corr);
  free(ctx);
  return 0;
}
