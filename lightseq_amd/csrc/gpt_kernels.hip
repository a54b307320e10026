// Kernels of the int8 GPT path: embedding, prompt-pass QKV split, the launchers of
// the reference's GPT kernel header (causal softmax over int32 scores, cache re-layout,
// greedy sampling, perplexity) and the fixed-stride greedy step the model itself runs.
//
// The model keeps keys and values in caches of fixed stride [batch, head, max_step, d]
// and token ids in [batch, max_step]: a generation step appends one column in place,
// where the reference re-lays out (copies) every cache and the whole id matrix per step.
#include "ls_device.h"
#include "ls_launch.h"
#include "sample_common.h"

#include <string>
#include <type_traits>

namespace lsh {

constexpr float kLogitThreshMin = -64.f;  // inference/kernels/transformerKernels.h:11

// ---------------------------------------------------------------------------------
// embedding (inference/kernels/gptKernels_int8.cc.cu:21-106); token_emb [vocab, hidden]
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
gpt_embedding_kernel(const int8_t* __restrict__ token_emb, const T* __restrict__ pos_emb,
                     const int* __restrict__ token_id, T* __restrict__ output, int padding_id,
                     int pos_offset, float dequant_scale, int seq_len, int hidden, int vocab) {
#pragma clang fp contract(off)
  const long pos = blockIdx.x;  // batch * seq_len + s
  const int s = (int)(pos % seq_len);
  int tid = token_id[pos];
  if (tid == padding_id) {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) TT<T>::st(output, pos * hidden + i, 0.f);
    return;
  }
  if (vocab > 0) tid = min(max(tid, 0), vocab - 1);  // never index outside the table
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = (float)token_emb[(long)tid * hidden + i] * dequant_scale +
                    TT<T>::ld(pos_emb, (long)(s + pos_offset) * hidden + i);
    TT<T>::st(output, pos * hidden + i, v);
  }
}

// The same for one position per sequence (a generation step): a workgroup per sequence, four
// elements per lane, no division; it also counts the token into real_seq_len (what
// gpt_count_tokens_kernel does in a launch of its own) and clears `zero_flag` when given, so a
// step spends one launch here instead of three.  Same arithmetic, same bits.
template <typename T>
__global__ void __launch_bounds__(256)
gpt_embedding_step_kernel(const int8_t* __restrict__ token_emb, const T* __restrict__ pos_emb,
                          const int* __restrict__ token_id, T* __restrict__ output,
                          int* real_seq_len, int* zero_flag, int padding_id, int pos,
                          float dequant_scale, int hidden, int vocab) {
#pragma clang fp contract(off)
  const int b = blockIdx.x;
  int tid = token_id[b];
  const bool pad = tid == padding_id;
  if (vocab > 0) tid = min(max(tid, 0), vocab - 1);  // never index outside the table
  if (threadIdx.x == 0) {
    if (!pad) real_seq_len[b] += 1;
    if (zero_flag != nullptr && b == 0) zero_flag[0] = 0;
  }
  for (int i = threadIdx.x * 4; i < hidden; i += blockDim.x * 4) {
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    if (!pad) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(token_emb + (long)tid * hidden + i);
      float p[4];
      ld4(pos_emb, (long)pos * hidden + i, p);
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = (float)unpack_i8(w, k) * dequant_scale + p[k];
    }
    st4(output, (long)b * hidden + i, o);
  }
}

// real_seq_len[b] += non-padding tokens of row b (the reference counts with atomics)
__global__ void __launch_bounds__(256)
gpt_count_tokens_kernel(const int* __restrict__ token_id, int* real_seq_len, int padding_id,
                        int seq_len) {
  __shared__ float red[16];
  const int b = blockIdx.x;
  float n = 0.f;
  for (int s = threadIdx.x; s < seq_len; s += blockDim.x)
    n += token_id[(long)b * seq_len + s] != padding_id ? 1.f : 0.f;
  n = block_sum(n, red);  // exact: seq_len is far below 2^24
  if (threadIdx.x == 0) real_seq_len[b] += (int)n;
}

template <typename T>
int gpt_embedding_i8I(int batch_size, int batch_seq_len, int hidden_size, hipStream_t s,
                      const int8_t* token_emb, const T* pos_emb, const int* token_id, T* output,
                      int* real_seq_len, int padding_id, int pos_offset, float dequant_scale,
                      int vocab_size, int max_step, int* zero_flag) {
  if (!token_emb || !pos_emb || !token_id || !output || !real_seq_len || batch_size <= 0 ||
      batch_seq_len <= 0 || hidden_size <= 0)
    return lsh_fail(LSH_ERR_INVALID, "ker_gpt_embedding_i8I: bad arguments");
  if (pos_offset < 0 || (max_step > 0 && pos_offset + batch_seq_len > max_step))
    return lsh_fail(LSH_ERR_INVALID, "ker_gpt_embedding_i8I: position outside the table");
  const bool aligned = ((reinterpret_cast<uintptr_t>(token_emb) | reinterpret_cast<uintptr_t>(pos_emb) |
                         reinterpret_cast<uintptr_t>(output)) & 15u) == 0;
  if (batch_seq_len == 1 && hidden_size % 4 == 0 && aligned) {
    gpt_embedding_step_kernel<T><<<batch_size, 256, 0, s>>>(
        token_emb, pos_emb, token_id, output, real_seq_len, zero_flag, padding_id, pos_offset,
        dequant_scale, hidden_size, vocab_size);
    return lsh_check_launch("gpt_embedding_step_kernel");
  }
  if (zero_flag != nullptr)
    if (int rc = fill_i32(zero_flag, 0, 1, s)) return rc;
  gpt_embedding_kernel<T><<<batch_size * batch_seq_len, 256, 0, s>>>(
      token_emb, pos_emb, token_id, output, padding_id, pos_offset, dequant_scale, batch_seq_len,
      hidden_size, vocab_size);
  if (int rc = lsh_check_launch("gpt_embedding_kernel")) return rc;
  gpt_count_tokens_kernel<<<batch_size, 256, 0, s>>>(token_id, real_seq_len, padding_id,
                                                     batch_seq_len);
  return lsh_check_launch("gpt_count_tokens_kernel");
}
template int gpt_embedding_i8I<float>(int, int, int, hipStream_t, const int8_t*, const float*,
                                      const int*, float*, int*, int, int, float, int, int, int*);
template int gpt_embedding_i8I<__half>(int, int, int, hipStream_t, const int8_t*, const __half*,
                                       const int*, __half*, int*, int, int, float, int, int, int*);

// ---------------------------------------------------------------------------------
// prompt pass: int8 QKV GEMM output [tokens, 3H] + bias -> requantised with the cache
// clip and written four ways in one pass:
//   q, k as fp16 *code values* [B, h, S, d]   (operands of the MFMA score product)
//   v dequantised to fp16      [B, h, S, d]   (code / quant_scale, the reference's d_v)
//   k, v int8 codes into the caches [B, h, max_step, d]
// Same arithmetic as ker_arrange_encself_qkv_i8I_i8O
// (inference/kernels/transformerKernels_int8.cc.cu:1185-1299).
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
gpt_arrange_qkv_prefill_kernel(const int8_t* __restrict__ ori_qkv,
                               const __half* __restrict__ qkv_bias, __half* __restrict__ q_codes,
                               __half* __restrict__ k_codes, __half* __restrict__ v_deq,
                               int8_t* __restrict__ k_cache, int8_t* __restrict__ v_cache,
                               int seq_len, int head_num, int d, int max_step,
                               float dequant_scale, float quant_scale) {
#pragma clang fp contract(off)
  const int H = head_num * d;
  const long tok = blockIdx.x;
  const int part = blockIdx.y;
  const long b = tok / seq_len;
  const int s = (int)(tok % seq_len);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float val = (float)ori_qkv[(tok * 3 + part) * H + i] * dequant_scale +
                      __half2float(qkv_bias[(long)part * H + i]);
    const int code = float2int8(val, quant_scale);
    const int head = i / d, dim = i % d;
    const long t = ((b * head_num + head) * seq_len + s) * d + dim;
    const long c = ((b * head_num + head) * max_step + s) * d + dim;
    if (part == 0) {
      q_codes[t] = __float2half_rn((float)code);
    } else if (part == 1) {
      k_codes[t] = __float2half_rn((float)code);
      k_cache[c] = (int8_t)code;
    } else {
      v_deq[t] = __float2half_rn((float)code / quant_scale);
      v_cache[c] = (int8_t)code;
    }
  }
}

int gpt_arrange_qkv_prefill_f16(int batch_token_num, int hidden_size, hipStream_t s,
                                const int8_t* ori_qkv, const __half* qkv_bias, __half* q_codes,
                                __half* k_codes, __half* v_deq, int8_t* k_cache, int8_t* v_cache,
                                int batch_seq_len, int dim_per_head, int head_num, int max_step,
                                float dequant_scale, float quant_scale) {
  if (!ori_qkv || !qkv_bias || !q_codes || !k_codes || !v_deq || !k_cache || !v_cache ||
      batch_token_num <= 0 || batch_seq_len <= 0 || batch_token_num % batch_seq_len != 0 ||
      hidden_size != dim_per_head * head_num || batch_seq_len > max_step)
    return lsh_fail(LSH_ERR_INVALID, "gpt_arrange_qkv_prefill: bad arguments");
  gpt_arrange_qkv_prefill_kernel<<<dim3(batch_token_num, 3), 256, 0, s>>>(
      ori_qkv, qkv_bias, q_codes, k_codes, v_deq, k_cache, v_cache, batch_seq_len, head_num,
      dim_per_head, max_step, dequant_scale, quant_scale);
  return lsh_check_launch("gpt_arrange_qkv_prefill_kernel");
}

// ---------------------------------------------------------------------------------
// causal softmax over int32 scores (inference/kernels/gptKernels_int8.cc.cu:192-250);
// one wavefront per (batch, head, query) row.  Rows of padded queries are written as
// zeros (the reference leaves them untouched).
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
softmax_gpt_i32I_kernel(const int32_t* __restrict__ corr, T* __restrict__ out,
                        const int* __restrict__ real_seq_len, long rows, int seq_len, int head_num,
                        float attn_scale, float dq) {
#pragma clang fp contract(off)
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int b = (int)(row / ((long)head_num * seq_len));
  const int qpos = (int)(row % seq_len);
  const int32_t* c = corr + row * seq_len;
  T* o = out + row * seq_len;
  if (qpos >= real_seq_len[b]) {
    for (int j = lane; j < seq_len; j += 64) TT<T>::st(o, j, 0.f);
    return;
  }
  float mx = kFloatInfNeg;
  for (int j = lane; j <= qpos; j += 64) mx = fmaxf(mx, (float)c[j] * attn_scale * dq * dq);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j <= qpos; j += 64) sum += __expf((float)c[j] * attn_scale * dq * dq - mx);
  sum = wave_sum(sum);
  for (int j = lane; j < seq_len; j += 64) {
    const float e = j <= qpos ? __expf((float)c[j] * attn_scale * dq * dq - mx) : 0.f;
    TT<T>::st(o, j, e / sum);
  }
}

template <typename T>
int correlation_softmax_gpt_i32I(int batch_size, int batch_seq_len, int head_num, hipStream_t s,
                                 const int32_t* correlation, T* output, const int* real_seq_len,
                                 float attn_scale, float dequant_scale) {
  if (!correlation || !output || !real_seq_len || batch_size <= 0 || batch_seq_len <= 0 ||
      head_num <= 0)
    return lsh_fail(LSH_ERR_INVALID, "ker_correlation_softmax_gpt_i32I: bad arguments");
  const long rows = (long)batch_size * head_num * batch_seq_len;
  softmax_gpt_i32I_kernel<T><<<(int)((rows + 3) / 4), 256, 0, s>>>(
      correlation, output, real_seq_len, rows, batch_seq_len, head_num, attn_scale,
      dequant_scale);
  return lsh_check_launch("softmax_gpt_i32I_kernel");
}
template int correlation_softmax_gpt_i32I<float>(int, int, int, hipStream_t, const int32_t*,
                                                 float*, const int*, float, float);
template int correlation_softmax_gpt_i32I<__half>(int, int, int, hipStream_t, const int32_t*,
                                                  __half*, const int*, float, float);

// ---------------------------------------------------------------------------------
// ker_attention_mask_weights_i32I (inference/kernels/gptKernels_int8.cc.cu:815-853): the
// soft-max of the last dst_seq_len query positions of a sequence over src_seq_len keys, each
// query seeing the keys up to its own position.  correlation / output [batch, head_num *
// dst_seq_len, src_seq_len]; a query at or beyond its sequence's real length leaves its output
// row untouched, as the reference's early return does.  The reference runs one thread per key
// (src_seq_len <= 1024); here a wavefront takes a row.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
attention_mask_weights_i32I_kernel(const int32_t* __restrict__ corr, T* __restrict__ out,
                                   const int* __restrict__ real_seq_len, long rows,
                                   int rows_per_batch, int dst_seq_len, int src_seq_len,
                                   float attn_scale, float dq) {
#pragma clang fp contract(off)
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int b = (int)(row / rows_per_batch);
  const int qpos = (int)(row % dst_seq_len) + src_seq_len - dst_seq_len;
  if (qpos >= real_seq_len[b]) return;
  const int32_t* c = corr + row * src_seq_len;
  T* o = out + row * src_seq_len;
  float mx = kFloatInfNeg;
  for (int j = lane; j <= qpos && j < src_seq_len; j += 64)
    mx = fmaxf(mx, (float)c[j] * attn_scale * dq * dq);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j <= qpos && j < src_seq_len; j += 64)
    sum += expf(fmaxf(kLogitThreshMin, (float)c[j] * attn_scale * dq * dq - mx));
  sum = wave_sum(sum);
  for (int j = lane; j < src_seq_len; j += 64) {
    const float e =
        j <= qpos ? expf(fmaxf(kLogitThreshMin, (float)c[j] * attn_scale * dq * dq - mx)) : 0.f;
    TT<T>::st(o, j, e / (sum + 1e-12f));  // epsilon: inference/kernels/transformerKernels.h:13
  }
}

template <typename T>
int attention_mask_weights_i32I(int batch_size, int dst_seq_len, int src_seq_len, int head_num,
                                hipStream_t s, const int32_t* correlation, T* output,
                                const int* real_seq_len, float attn_scale, float dequant_scale) {
  if (!correlation || !output || !real_seq_len || batch_size <= 0 || dst_seq_len <= 0 ||
      src_seq_len < dst_seq_len || head_num <= 0)
    return lsh_fail(LSH_ERR_INVALID, "ker_attention_mask_weights_i32I: bad arguments");
  if (src_seq_len > 1024)  // the reference launches src_seq_len threads per block
    return lsh_fail(LSH_ERR_INVALID, "ker_attention_mask_weights_i32I: src_seq_len above 1024");
  const int rows_per_batch = head_num * dst_seq_len;
  const long rows = (long)batch_size * rows_per_batch;
  attention_mask_weights_i32I_kernel<T><<<(int)((rows + 3) / 4), 256, 0, s>>>(
      correlation, output, real_seq_len, rows, rows_per_batch, dst_seq_len, src_seq_len,
      attn_scale, dequant_scale);
  return lsh_check_launch("attention_mask_weights_i32I_kernel");
}
template int attention_mask_weights_i32I<float>(int, int, int, int, hipStream_t, const int32_t*,
                                                float*, const int*, float, float);
template int attention_mask_weights_i32I<__half>(int, int, int, int, hipStream_t, const int32_t*,
                                                 __half*, const int*, float, float);

// batched int8 q.K^T of the prompt pass (inference/model/quant_gpt_encoder.cc.cu:498-505)
// for callers of the unfused launchers: scores[bh, i, j] = sum_d q[bh,i,d] * k[bh,j,d]
__global__ void __launch_bounds__(256)
gpt_scores_i8_kernel(const int8_t* __restrict__ q, const int8_t* __restrict__ k,
                     int32_t* __restrict__ scores, long rows, int seq_len, int d) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const long bh = row / seq_len;
  const int8_t* qp = q + row * d;
  for (int j = lane; j < seq_len; j += 64) {
    const int8_t* kp = k + (bh * seq_len + j) * d;
    int acc = 0;
    for (int t = 0; t < d; ++t) acc += (int)qp[t] * (int)kp[t];
    scores[row * seq_len + j] = acc;
  }
}

int gpt_scores_i8(const int8_t* q, const int8_t* k, int32_t* scores, int batch_head_num,
                  int batch_seq_len, int dim_per_head, hipStream_t s) {
  if (!q || !k || !scores || batch_head_num <= 0 || batch_seq_len <= 0 || dim_per_head <= 0)
    return lsh_fail(LSH_ERR_INVALID, "gpt_scores_i8: bad arguments");
  const long rows = (long)batch_head_num * batch_seq_len;
  gpt_scores_i8_kernel<<<(int)((rows + 3) / 4), 256, 0, s>>>(q, k, scores, rows, batch_seq_len,
                                                             dim_per_head);
  return lsh_check_launch("gpt_scores_i8_kernel");
}

// ---------------------------------------------------------------------------------
// ker_arrange_qkv_with_cache_i8I_i8O (inference/kernels/gptKernels_int8.cc.cu:658-812):
// one new token per sequence; caches re-laid out from [B, h, S-1, d] to [B, h, S, d]
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
arrange_qkv_with_cache_kernel(const int8_t* __restrict__ ori_qkv, const T* __restrict__ qkv_bias,
                              int8_t* __restrict__ new_q, int8_t* __restrict__ new_k,
                              const int8_t* __restrict__ k_cache, int8_t* __restrict__ new_v,
                              const int8_t* __restrict__ v_cache, int seq_len, int d, int head_num,
                              float dequant_scale, float quant_scale) {
#pragma clang fp contract(off)
  const int H = head_num * d;
  const long b = blockIdx.x / seq_len;
  const int t = blockIdx.x % seq_len;
  const int part = blockIdx.y;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const int head = i / d, dim = i % d;
    const long target = ((b * head_num + head) * seq_len + t) * d + dim;
    if (t < seq_len - 1) {
      if (part == 0) return;
      const long old = ((b * head_num + head) * (seq_len - 1) + t) * d + dim;
      if (part == 1) new_k[target] = k_cache[old];
      else new_v[target] = v_cache[old];
    } else {
      const float val = (float)ori_qkv[(b * 3 + part) * H + i] * dequant_scale +
                        TT<T>::ld(qkv_bias, (long)part * H + i);
      const int8_t qv = (int8_t)float2int8(val, quant_scale);
      if (part == 0) new_q[(b * head_num + head) * d + dim] = qv;
      else if (part == 1) new_k[target] = qv;
      else new_v[target] = qv;
    }
  }
}

template <typename T>
int arrange_qkv_with_cache_i8I_i8O(int batch_token_num, int hidden_size, hipStream_t s,
                                   const int8_t* ori_qkv, const T* qkv_bias, int8_t* new_q,
                                   int8_t* new_k, const int8_t* k_cache, int8_t* new_v,
                                   const int8_t* v_cache, int batch_seq_len, int dim_per_head,
                                   int head_num, float dequant_scale, float quant_scale) {
  if (!ori_qkv || !qkv_bias || !new_q || !new_k || !new_v || batch_token_num <= 0 ||
      batch_seq_len <= 0 || batch_token_num % batch_seq_len != 0 ||
      hidden_size != dim_per_head * head_num || (batch_seq_len > 1 && (!k_cache || !v_cache)))
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_qkv_with_cache_i8I_i8O: bad arguments");
  if (new_k == k_cache || new_v == v_cache)
    return lsh_fail(LSH_ERR_INVALID,
                    "ker_arrange_qkv_with_cache_i8I_i8O: old and new cache must differ");
  arrange_qkv_with_cache_kernel<T><<<dim3(batch_token_num, 3), 256, 0, s>>>(
      ori_qkv, qkv_bias, new_q, new_k, k_cache, new_v, v_cache, batch_seq_len, dim_per_head,
      head_num, dequant_scale, quant_scale);
  return lsh_check_launch("arrange_qkv_with_cache_kernel");
}
template int arrange_qkv_with_cache_i8I_i8O<float>(int, int, hipStream_t, const int8_t*,
                                                   const float*, int8_t*, int8_t*, const int8_t*,
                                                   int8_t*, const int8_t*, int, int, int, float,
                                                   float);
template int arrange_qkv_with_cache_i8I_i8O<__half>(int, int, hipStream_t, const int8_t*,
                                                    const __half*, int8_t*, int8_t*,
                                                    const int8_t*, int8_t*, const int8_t*, int, int,
                                                    int, float, float);

// ---------------------------------------------------------------------------------
// greedy sampling.  The dequantisation code * scale (scale > 0) is monotone, so the
// arg-max runs on the int8 codes; ties go to the lowest token id (the reference lets
// racing stores decide).
// ---------------------------------------------------------------------------------
// First maximum of a row of int8 logits (lowest id on ties), the same in every thread.  A
// candidate is the key (code + 128) << 20 | (2^20 - 1 - id), so the arg-max is one integer
// maximum: over a wavefront by DPP permutations and lane reads, over the workgroup through LDS
// with one barrier.  vocab <= 2^20.
// The row starts anywhere (an odd vocabulary), so it is read as the 16-byte pieces that lie
// wholly inside it -- four per thread requested together, the index clamped instead of the load
// predicated -- plus at most 15 bytes before and 15 after them, one per thread of the first
// wavefront.  No branch sits between the loads and none around them: per element it is one
// bit-field extract, one shift-add and one maximum (the kernel's length is its instruction
// count; the byte-by-byte handling of partial pieces this replaces was 3000 instructions).
__device__ __forceinline__ int block_argmax_i8(const int8_t* __restrict__ lr, int vocab,
                                               int* red /*[32]*/) {
  constexpr int kIdBits = 20, kIdMask = (1 << kIdBits) - 1;
  const int t = threadIdx.x;
  const int a = (int)(reinterpret_cast<uintptr_t>(lr) & 15u);
  const int head = min((16 - a) & 15, vocab);  // elements before the first aligned piece
  const int8_t* body = lr + head;              // 16-byte aligned
  const int nfull = (vocab - head) >> 4;       // whole pieces inside the row
  const int tail0 = head + (nfull << 4);       // first element behind them
  // head (threads 0..15) and tail (threads 16..31) elements, one byte each
  const int ev = t < 16 ? t : tail0 + (t - 16);
  const bool eon = t < 16 ? t < head : (t < 32 && ev < vocab);
  const int ec = lr[eon ? ev : 0];
  int key = eon ? (((ec + 128) << kIdBits) | (kIdMask - ev)) : 0;  // 0: below every real key
  for (int p0 = 0; p0 < nfull; p0 += 4 * (int)blockDim.x) {
    uint4 w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      w[u] = *reinterpret_cast<const uint4*>(
          body + (long)min(p0 + u * (int)blockDim.x + t, nfull - 1) * 16);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = p0 + u * (int)blockDim.x + t;
      const int base = kIdMask - (head + p * 16);  // id part of the piece's first element
      const uint32_t ws[4] = {w[u].x ^ 0x80808080u, w[u].y ^ 0x80808080u, w[u].z ^ 0x80808080u,
                              w[u].w ^ 0x80808080u};  // code + 128 in every byte
      int kp = 0;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int c = (int)__builtin_amdgcn_ubfe(ws[e >> 2], 8 * (e & 3), 8);
        kp = max(kp, (c << kIdBits) + (base - e));
      }
      key = p < nfull ? max(key, kp) : key;
    }
  }
  auto max_dpp = [](int x, auto ctrl) {
    return max(x, __builtin_amdgcn_update_dpp(0, x, decltype(ctrl)::value, 0xf, 0xf, false));
  };
  key = max_dpp(key, std::integral_constant<int, 0xB1>());   // lane ^ 1
  key = max_dpp(key, std::integral_constant<int, 0x4E>());   // lane ^ 2
  key = max_dpp(key, std::integral_constant<int, 0x141>());  // the other quad of 8
  key = max_dpp(key, std::integral_constant<int, 0x140>());  // the other half of 16
  key = max(max(__builtin_amdgcn_readlane(key, 0), __builtin_amdgcn_readlane(key, 16)),
            max(__builtin_amdgcn_readlane(key, 32), __builtin_amdgcn_readlane(key, 48)));
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  if (lane == 0) red[wid] = key;
  __syncthreads();
  key = red[0];
  for (int w2 = 1; w2 < nw; ++w2) key = max(key, red[w2]);
  return kIdMask - (key & kIdMask);
}

// ker_topk_sample_i8I<1> (inference/kernels/gptKernels_int8.cc.cu:252-463): ids re-laid
// out from [batch, seq_len] to [batch, seq_len + 1], sampled ids also behind the old array
__global__ void __launch_bounds__(1024)
topk_sample_greedy_kernel(const int8_t* __restrict__ logits, int* old_input_ids,
                          int* __restrict__ new_input_ids, int vocab, int seq_len,
                          int logits_seq_len, int* unfinished, int eos_id) {
  __shared__ int red[32];
  const int b = blockIdx.x;
  const bool ended = old_input_ids[(long)b * seq_len + seq_len - 1] == eos_id;
  for (int t = threadIdx.x; t < seq_len; t += blockDim.x)
    new_input_ids[(long)b * (seq_len + 1) + t] = old_input_ids[(long)b * seq_len + t];
  int tok = eos_id;
  if (!ended) {
    const int8_t* lr = logits + ((long)b * logits_seq_len + logits_seq_len - 1) * vocab;
    tok = block_argmax_i8(lr, vocab, red);
  }
  if (threadIdx.x == 0) {
    if (!ended && tok != eos_id) unfinished[0] = 1;  // every writer stores the same value
    new_input_ids[(long)b * (seq_len + 1) + seq_len] = tok;
  }
}

// second pass: sampled ids behind the old array, after every block has read its old row
__global__ void topk_sample_tail_kernel(int* old_input_ids, const int* __restrict__ new_input_ids,
                                        int batch, int seq_len) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < batch)
    old_input_ids[(long)batch * seq_len + b] = new_input_ids[(long)b * (seq_len + 1) + seq_len];
}

static int sample_ids(int batch_size, int batch_seq_len, int logits_seq_len, hipStream_t s,
                      const int8_t* logits, int* old_input_ids, int* new_input_ids, int vocab_size,
                      int k, float p, int* unfinished, void* state, int eos_id,
                      float dequant_scale, const char* who);

int topk_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len, hipStream_t s,
                    const int8_t* logits, int* old_input_ids, int* new_input_ids,
                    int vocab_size, int k, int* unfinished, int eos_id, void* state,
                    float dequant_scale) {
  if (!logits || !old_input_ids || !new_input_ids || !unfinished || batch_size <= 0 ||
      batch_seq_len <= 0 || logits_seq_len <= 0 || vocab_size <= 0)
    return lsh_fail(LSH_ERR_INVALID, "ker_topk_sample_i8I: bad arguments");
  if (k != 1) {
    if (k == 2 || k == 4 || k == 8 || k == 16 || k == 32)
      return sample_ids(batch_size, batch_seq_len, logits_seq_len, s, logits, old_input_ids,
                        new_input_ids, vocab_size, k, 0.f, unfinished, state, eos_id,
                        dequant_scale, "ker_topk_sample_i8I");
    return lsh_fail(LSH_ERR_INVALID, "topk argument should be in [1,2,4,8,16,32]");
  }
  if (vocab_size > (1 << 20))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "ker_topk_sample_i8I: vocabulary above 2^20 ids");
  topk_sample_greedy_kernel<<<batch_size, 1024, 0, s>>>(logits, old_input_ids, new_input_ids,
                                                        vocab_size, batch_seq_len, logits_seq_len,
                                                        unfinished, eos_id);
  if (int rc = lsh_check_launch("topk_sample_greedy_kernel")) return rc;
  topk_sample_tail_kernel<<<(batch_size + 255) / 256, 256, 0, s>>>(old_input_ids, new_input_ids,
                                                                   batch_size, batch_seq_len);
  return lsh_check_launch("topk_sample_tail_kernel");
}

// the model's step: ids [batch, max_step] in place, logits [batch, vocab] of the last
// position; writes column cur_len, the step's input ids and the unfinished flag
__global__ void __launch_bounds__(1024)
gpt_greedy_step_kernel(const int8_t* __restrict__ logits, int* ids, int* __restrict__ last_ids,
                       int vocab, int max_step, int cur_len, int* unfinished, int eos_id) {
  __shared__ int red[32];
  const int b = blockIdx.x;
  const bool ended = ids[(long)b * max_step + cur_len - 1] == eos_id;
  int tok = eos_id;
  if (!ended) tok = block_argmax_i8(logits + (long)b * vocab, vocab, red);
  if (threadIdx.x == 0) {
    if (!ended && tok != eos_id) unfinished[0] = 1;
    ids[(long)b * max_step + cur_len] = tok;
    last_ids[b] = tok;
  }
}

int gpt_greedy_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size, int max_step,
                    int cur_len, int batch_size, int* unfinished, int eos_id, hipStream_t s) {
  if (!logits || !ids || !last_ids || !unfinished || batch_size <= 0 || vocab_size <= 0 ||
      cur_len <= 0 || cur_len >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "gpt_greedy_step: bad arguments");
  if (vocab_size > (1 << 20))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "gpt_greedy_step: vocabulary above 2^20 ids");
  gpt_greedy_step_kernel<<<batch_size, 1024, 0, s>>>(logits, ids, last_ids, vocab_size, max_step,
                                                     cur_len, unfinished, eos_id);
  return lsh_check_launch("gpt_greedy_step_kernel");
}

// ---------------------------------------------------------------------------------
// random sampling: ker_topk_sample_i8I<k>, k > 1 (inference/kernels/gptKernels_int8.cc.cu:252-
// 420) and ker_topp_sample_i8I (:465-640) as they act with the 1024 threads per block the model
// launches them with: thread t owns the vocabulary ids congruent to t modulo 1024 (a class),
// the candidate set holds at most one id per class -- the first one of the largest
// exp(max(logit - max, -64)) among the class's ids at or above a threshold -- and one uniform
// number picks the first class, in thread order, whose cumulative probability reaches it.
// Top-k: the threshold is the rough k-th largest class maximum (kernels/common.h:118-137:
// maxima of the 32 warps of 32 threads, maximum over the warps that agree modulo k, minimum
// over the k groups).  Top-p: the reference compares every thread's prefix sum with a threshold
// that only its last thread assigns (:533-539), which defines nothing; built here is what it
// intends: class maxima in descending order, exps, inclusive prefix, and the threshold is the
// smallest maximum whose prefix stays within p of the total (at least the largest).
// The dequantisation code * scale (scale > 0) is monotone, so maxima, thresholds and the order
// of candidates run on the int8 codes; exps and probabilities are float as in the reference.
// The uniform numbers: the reference draws them from a cuRAND state seeded with clock()
// (kernels/transformerKernels.cc.cu:2270-2274); here they are Philox4x32-10 words (key = seed,
// counter = (draw, 0, row, 0), word 0) mapped to (0, 1] as curand_uniform maps 32 bits, with
// the state {seed, row, draws} per sequence in device memory, advanced by the kernel.
// ---------------------------------------------------------------------------------
__global__ void sample_state_setup_kernel(SampleState* st, int n, unsigned long long seed) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) st[i] = SampleState{seed, (unsigned)i, 0u};
}

int sample_state_setup(void* state, int n, unsigned long long seed, hipStream_t s) {
  if (!state || n <= 0 || (reinterpret_cast<uintptr_t>(state) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "rng_setup: needs a 16-byte aligned state array");
  sample_state_setup_kernel<<<(n + 255) / 256, 256, 0, s>>>(static_cast<SampleState*>(state), n,
                                                            seed);
  return lsh_check_launch("sample_state_setup_kernel");
}

// The 16 consecutive ids a thread reads per piece belong to 16 classes that do not change from
// piece to piece (16 * 1024 is a multiple of 1024), so a thread reduces in registers and
// touches LDS 16 times at the end.  f(e, v, c): slot e of the thread, id v, code c.
template <typename F>
__device__ __forceinline__ void sample_scan_row(const int8_t* __restrict__ lr, int vocab, F f) {
  const int a = (int)(reinterpret_cast<uintptr_t>(lr) & 15u);
  const int8_t* base = lr - a;
  const int pieces = (vocab + a + 15) >> 4;
  for (int p = threadIdx.x; p < pieces; p += kSampleThreads) {
    const int v0 = p * 16 - a;
    if (v0 >= 0 && v0 + 16 <= vocab) {
      const uint4 w = *reinterpret_cast<const uint4*>(base + (long)p * 16);
      const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int e = 0; e < 16; ++e) f(e, v0 + e, unpack_i8(ws[e >> 2], e & 3));
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e)
        if (v0 + e >= 0 && v0 + e < vocab) f(e, v0 + e, (int)lr[v0 + e]);
    }
  }
}

// One row; every thread returns the sampled id.  k > 1: top-k, k == 0: top-p with p.
__device__ int sample_row(const int8_t* __restrict__ lr, int vocab, int k, float p, float scale,
                          SampleState* st, SampleShared& sh) {
  const int t = threadIdx.x;
  const int a = (int)(reinterpret_cast<uintptr_t>(lr) & 15u);
  const int cls0 = (16 * t - a) & (kSampleThreads - 1);  // class of the thread's slot 0
  sh.cls[t] = -129;
  if (t < 260) sh.hist[t] = 0;
  if (t == 0) sh.x = sample_draw_uniform(st);
  __syncthreads();
  {
    int m[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) m[e] = -129;
    sample_scan_row(lr, vocab, [&](int e, int, int c) { m[e] = max(m[e], c); });
#pragma unroll
    for (int e = 0; e < 16; ++e)
      if (m[e] > -129) atomicMax(&sh.cls[(cls0 + e) & (kSampleThreads - 1)], m[e]);
  }
  __syncthreads();
  const int cm = sh.cls[t];
  const int gmax = (int)block_max((float)cm, sh.red);
  const float mx = (float)gmax * scale;
  if (k > 0) {
    // rough k-th largest class maximum
    if (t < 32) {
      int w = sh.cls[32 * t];
      for (int l = 1; l < 32; ++l) w = max(w, sh.cls[32 * t + l]);
      sh.hist[t] = w;
    }
    __syncthreads();
    if (t == 0) {
      int best = 127;
      for (int g = 0; g < k; ++g) {
        int w = sh.hist[g];
        for (int j = g + k; j < 32; j += k) w = max(w, sh.hist[j]);
        best = min(best, w);
      }
      sh.thr = best;
    }
  } else {
    // classes per maximum code, exp of every code, then one thread walks the codes downwards
    atomicAdd(&sh.hist[cm + 129], 1);
    if (t < 257)
      sh.pf[t] = expf(fmaxf((float)(t - 129) * scale - mx, kLogitThreshMin));  // t = code + 129
    __syncthreads();
    if (t == 0) {
      // an empty class holds -inf in the reference: exp(-64) each
      float total = (float)sh.hist[0] * expf(kLogitThreshMin);
      for (int c = gmax; c >= -128; --c) total += (float)sh.hist[c + 129] * sh.pf[c + 129];
      const float limit = p * total;
      float pre = 0.f;
      int thr = gmax;
      for (int c = gmax; c >= -128; --c) {
        const int n = sh.hist[c + 129];
        if (n == 0) continue;
        if (pre + sh.pf[c + 129] > limit) break;
        thr = c;
        pre += (float)n * sh.pf[c + 129];
      }
      sh.thr = thr;
    }
  }
  __syncthreads();
  const int thr = sh.thr;
  sh.cls[t] = 0;  // candidate keys: (rank << 20) | (2^20 - 1 - id); 0 = none
  __syncthreads();
  {
    // rank: 1 where the exp is clamped (all such ids tie: the first one wins), code + 130 else
    int key[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) key[e] = 0;
    sample_scan_row(lr, vocab, [&](int e, int v, int c) {
      if (c >= thr) {
        const bool clamped = (float)c * scale - mx < kLogitThreshMin;
        key[e] = max(key[e], ((clamped ? 1 : c + 130) << kSampleIdBits) | (kSampleIdMask - v));
      }
    });
#pragma unroll
    for (int e = 0; e < 16; ++e)
      if (key[e] != 0) atomicMax(&sh.cls[(cls0 + e) & (kSampleThreads - 1)], key[e]);
  }
  __syncthreads();
  const int key = sh.cls[t];
  const int rank = key >> kSampleIdBits;
  const int my_id = key == 0 ? vocab : kSampleIdMask - (key & kSampleIdMask);
  const float ex = key == 0 ? 0.f
                            : expf(rank == 1 ? kLogitThreshMin
                                             : fmaxf((float)(rank - 130) * scale - mx, kLogitThreshMin));
  return sample_pick(ex, my_id, sh);
}

// ker_topk_sample_i8I<k> / ker_topp_sample_i8I: ids re-laid out from [batch, seq_len] to
// [batch, seq_len + 1] (the sampled ids behind the old array by topk_sample_tail_kernel)
__global__ void __launch_bounds__(kSampleThreads)
sample_ids_kernel(const int8_t* __restrict__ logits, int* old_input_ids,
                  int* __restrict__ new_input_ids, int vocab, int seq_len, int logits_seq_len,
                  int* unfinished, int eos_id, int k, float p, float scale, SampleState* st) {
  __shared__ SampleShared sh;
  const int b = blockIdx.x;
  const bool ended = old_input_ids[(long)b * seq_len + seq_len - 1] == eos_id;
  for (int t = threadIdx.x; t < seq_len; t += blockDim.x)
    new_input_ids[(long)b * (seq_len + 1) + t] = old_input_ids[(long)b * seq_len + t];
  int tok = eos_id;
  if (!ended)
    tok = sample_row(logits + ((long)b * logits_seq_len + logits_seq_len - 1) * vocab, vocab, k, p,
                     scale, st + b, sh);
  if (threadIdx.x == 0) {
    if (!ended && tok != eos_id) unfinished[0] = 1;
    new_input_ids[(long)b * (seq_len + 1) + seq_len] = tok;
  }
}

static int sample_ids(int batch_size, int batch_seq_len, int logits_seq_len, hipStream_t s,
                      const int8_t* logits, int* old_input_ids, int* new_input_ids, int vocab_size,
                      int k, float p, int* unfinished, void* state, int eos_id,
                      float dequant_scale, const char* who) {
  if (!state || (reinterpret_cast<uintptr_t>(state) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, (std::string(who) + ": random sampling needs the generator "
                                                         "state array (lsh_rng_setup)").c_str());
  if (!(dequant_scale > 0.f))
    return lsh_fail(LSH_ERR_INVALID, (std::string(who) + ": dequant_scale must be positive").c_str());
  if (vocab_size > (1 << kSampleIdBits))
    return lsh_fail(LSH_ERR_UNSUPPORTED, (std::string(who) + ": vocabulary above 2^20 ids").c_str());
  sample_ids_kernel<<<batch_size, kSampleThreads, 0, s>>>(
      logits, old_input_ids, new_input_ids, vocab_size, batch_seq_len, logits_seq_len, unfinished,
      eos_id, k, p, dequant_scale, static_cast<SampleState*>(state));
  if (int rc = lsh_check_launch("sample_ids_kernel")) return rc;
  topk_sample_tail_kernel<<<(batch_size + 255) / 256, 256, 0, s>>>(old_input_ids, new_input_ids,
                                                                   batch_size, batch_seq_len);
  return lsh_check_launch("topk_sample_tail_kernel");
}

int topp_sample_i8I(int batch_size, int batch_seq_len, int logits_seq_len, hipStream_t s,
                    const int8_t* logits, int* old_input_ids, int* new_input_ids, int vocab_size,
                    float p, int* unfinished, void* state, int eos_id, float dequant_scale) {
  if (!logits || !old_input_ids || !new_input_ids || !unfinished || batch_size <= 0 ||
      batch_seq_len <= 0 || logits_seq_len <= 0 || vocab_size <= 0 || !(p > 0.f) || p > 1.f)
    return lsh_fail(LSH_ERR_INVALID, "ker_topp_sample_i8I: bad arguments");
  return sample_ids(batch_size, batch_seq_len, logits_seq_len, s, logits, old_input_ids,
                    new_input_ids, vocab_size, 0, p, unfinished, state, eos_id, dequant_scale,
                    "ker_topp_sample_i8I");
}

// the model's step with random sampling: as gpt_greedy_step_kernel
__global__ void __launch_bounds__(kSampleThreads)
gpt_sample_step_kernel(const int8_t* __restrict__ logits, int* ids, int* __restrict__ last_ids,
                       int vocab, int max_step, int cur_len, int* unfinished, int eos_id, int k,
                       float p, float scale, SampleState* st) {
  __shared__ SampleShared sh;
  const int b = blockIdx.x;
  const bool ended = ids[(long)b * max_step + cur_len - 1] == eos_id;
  int tok = eos_id;
  if (!ended) tok = sample_row(logits + (long)b * vocab, vocab, k, p, scale, st + b, sh);
  if (threadIdx.x == 0) {
    if (!ended && tok != eos_id) unfinished[0] = 1;
    ids[(long)b * max_step + cur_len] = tok;
    last_ids[b] = tok;
  }
}

int gpt_sample_step(const int8_t* logits, int* ids, int* last_ids, int vocab_size, int max_step,
                    int cur_len, int batch_size, int* unfinished, int eos_id, int k, float p,
                    float dequant_scale, void* state, hipStream_t s) {
  if (!logits || !ids || !last_ids || !unfinished || !state || batch_size <= 0 ||
      vocab_size <= 0 || cur_len <= 0 || cur_len >= max_step || !(dequant_scale > 0.f) ||
      (reinterpret_cast<uintptr_t>(state) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "gpt_sample_step: bad arguments");
  if (k != 0 && k != 2 && k != 4 && k != 8 && k != 16 && k != 32)
    return lsh_fail(LSH_ERR_INVALID, "topk argument should be in [1,2,4,8,16,32]");
  if (k == 0 && (!(p > 0.f) || p > 1.f))
    return lsh_fail(LSH_ERR_INVALID, "gpt_sample_step: topp outside (0, 1]");
  if (vocab_size > (1 << kSampleIdBits))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "gpt_sample_step: vocabulary above 2^20 ids");
  gpt_sample_step_kernel<<<batch_size, kSampleThreads, 0, s>>>(
      logits, ids, last_ids, vocab_size, max_step, cur_len, unfinished, eos_id, k, p,
      dequant_scale, static_cast<SampleState*>(state));
  return lsh_check_launch("gpt_sample_step_kernel");
}

// ---------------------------------------------------------------------------------
// perplexity (inference/kernels/gptKernels_int8.cc.cu:108-190).  The per-position terms of a
// sequence are added in ascending position order, so the sum has a fixed order (the reference
// adds them with float atomics).  With a workspace of batch * seq_len floats every (sequence,
// position) pair gets its own workgroup and a second kernel adds a sequence's terms in order;
// without one a workgroup per sequence walks its positions.  Both give the same bits.
// ---------------------------------------------------------------------------------
// -log p(next token) / (len - 1) of position s of sequence b, the same in every thread
__device__ __forceinline__ float ppl_term(const int8_t* __restrict__ logits,
                                          const int* __restrict__ input_ids, int b, int s, int len,
                                          int vocab, int seq_len, float dq, float* red) {
#pragma clang fp contract(off)
  const long tok = (long)b * seq_len + s;
  const int8_t* lr = logits + tok * vocab;
  float mx = kFloatInfNeg;
  for (int v = threadIdx.x; v < vocab; v += blockDim.x) mx = fmaxf(mx, (float)lr[v] * dq);
  mx = block_max(mx, red);
  float se = 0.f;
  for (int v = threadIdx.x; v < vocab; v += blockDim.x)
    se += __expf(fmaxf((float)lr[v] * dq - mx, kLogitThreshMin));
  se = block_sum(se, red);
  int target = input_ids[tok + 1];
  target = min(max(target, 0), vocab - 1);
  const float log_prob = ((float)lr[target] * dq - mx - logf(se)) / (float)(len - 1);
  return -log_prob;
}

__global__ void __launch_bounds__(1024)
ppl_kernel(const int8_t* __restrict__ logits, const int* __restrict__ input_ids,
           const int* __restrict__ real_seq_len, float* ppl, int vocab, int seq_len, float dq) {
  __shared__ float red[16];
  const int b = blockIdx.x;
  const int len = real_seq_len[b];
  float total = 0.f;
  for (int s = 0; s < seq_len && s < len - 1; ++s)
    total += ppl_term(logits, input_ids, b, s, len, vocab, seq_len, dq, red);
  if (threadIdx.x == 0) ppl[b] += total;
}

// grid (seq_len, batch): terms[b * seq_len + s]
__global__ void __launch_bounds__(1024)
ppl_terms_kernel(const int8_t* __restrict__ logits, const int* __restrict__ input_ids,
                 const int* __restrict__ real_seq_len, float* __restrict__ terms, int vocab,
                 int seq_len, float dq) {
  __shared__ float red[16];
  const int b = blockIdx.y, s = blockIdx.x;
  const int len = real_seq_len[b];
  if (s >= len - 1) return;  // (uniform: no term, nothing read by the sum)
  const float t = ppl_term(logits, input_ids, b, s, len, vocab, seq_len, dq, red);
  if (threadIdx.x == 0) terms[(long)b * seq_len + s] = t;
}

__global__ void ppl_sum_kernel(const float* __restrict__ terms,
                               const int* __restrict__ real_seq_len, float* ppl, int batch,
                               int seq_len) {
#pragma clang fp contract(off)
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch) return;
  const int len = real_seq_len[b];
  float total = 0.f;
  for (int s = 0; s < seq_len && s < len - 1; ++s) total += terms[(long)b * seq_len + s];
  ppl[b] += total;
}

int ppl_i8I(int batch_size, int batch_seq_len, hipStream_t s, const int8_t* logits,
            const int* input_ids, const int* real_seq_len, float* ppl, int vocab_size,
            float dequant_scale, float* workspace) {
  if (!logits || !input_ids || !real_seq_len || !ppl || batch_size <= 0 || batch_seq_len <= 0 ||
      vocab_size <= 0)
    return lsh_fail(LSH_ERR_INVALID, "ker_ppl_i8I: bad arguments");
  if (workspace != nullptr && batch_size <= 65535) {
    ppl_terms_kernel<<<dim3(batch_seq_len, batch_size), 1024, 0, s>>>(
        logits, input_ids, real_seq_len, workspace, vocab_size, batch_seq_len, dequant_scale);
    if (int rc = lsh_check_launch("ppl_terms_kernel")) return rc;
    ppl_sum_kernel<<<(batch_size + 63) / 64, 64, 0, s>>>(workspace, real_seq_len, ppl, batch_size,
                                                         batch_seq_len);
    return lsh_check_launch("ppl_sum_kernel");
  }
  ppl_kernel<<<batch_size, 1024, 0, s>>>(logits, input_ids, real_seq_len, ppl, vocab_size,
                                         batch_seq_len, dequant_scale);
  return lsh_check_launch("ppl_kernel");
}

}  // namespace lsh
