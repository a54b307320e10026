// Decoder-step kernels: target embedding, the int8 self-attention against the
// K/V cache, and the fp16 attention over the projected encoder output.
//
// One decoding step handles rows = batch * beam_size query vectors, so every kernel
// here is small and latency-bound: the layout goal is few launches and coalesced
// rows, not tiling.  A wavefront owns one (row, head) pair in the attention kernels;
// all cross-lane traffic is wave reductions, and sums run in a fixed order so that a
// step is reproducible bit for bit.
#include "dec_attend.h"
#include "ls_device.h"
#include "ls_launch.h"

namespace lsh {

// ---------------------------------------------------------------------------------
// target embedding (inference/kernels/embKernels_int8.cc.cu:158-200)
// ---------------------------------------------------------------------------------
template <typename T, bool VOCAB_MAJOR>
__global__ void __launch_bounds__(256)
dec_emb_kernel(const int8_t* __restrict__ token_emb, const T* __restrict__ pos_emb,
               const int* __restrict__ tokens, T* __restrict__ out, int rows, int hidden,
               int vocab, int step, int max_step, float scale) {
#pragma clang fp contract(off)
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)rows * hidden) return;
  const int r = (int)(idx / hidden), i = (int)(idx % hidden);
  int token = tokens[(long)r * max_step + step];
  token = min(max(token, 0), vocab - 1);  // never index outside the table
  const int8_t e =
      VOCAB_MAJOR ? token_emb[(long)token * hidden + i] : token_emb[(long)i * vocab + token];
  const float v = (float)e * scale + TT<T>::ld(pos_emb, (long)step * hidden + i);
  TT<T>::st(out, idx, v);
}

template <typename T>
int dec_emb_i8I(const int8_t* token_emb, const T* pos_emb, const int* tokens, T* output,
                int batch_size, int beam_size, int hidden_dim, int vocab_size, int step,
                int max_step, hipStream_t s, float dequant_scale, bool scaled, bool vocab_major) {
  if (!token_emb || !pos_emb || !tokens || !output || batch_size <= 0 || beam_size <= 0 ||
      hidden_dim <= 0 || vocab_size <= 0 || max_step <= 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_dec_emb_i8I: bad arguments");
  if (step < 0 || step >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "violate step < max_step");
  const int rows = batch_size * beam_size;
  float scale = dequant_scale;
  if (scaled) scale *= sqrtf((float)hidden_dim);
  const long n = (long)rows * hidden_dim;
  const int grid = (int)((n + 255) / 256);
  if (vocab_major)
    dec_emb_kernel<T, true><<<grid, 256, 0, s>>>(token_emb, pos_emb, tokens, output, rows,
                                                 hidden_dim, vocab_size, step, max_step, scale);
  else
    dec_emb_kernel<T, false><<<grid, 256, 0, s>>>(token_emb, pos_emb, tokens, output, rows,
                                                  hidden_dim, vocab_size, step, max_step, scale);
  return lsh_check_launch("dec_emb_kernel");
}
template int dec_emb_i8I<float>(const int8_t*, const float*, const int*, float*, int, int, int,
                                int, int, int, hipStream_t, float, bool, bool);
template int dec_emb_i8I<__half>(const int8_t*, const __half*, const int*, __half*, int, int, int,
                                 int, int, int, hipStream_t, float, bool, bool);

// ---------------------------------------------------------------------------------
// split QKV of the current step: q -> [rows, H] int8, k / v -> cache slot `step_id`
// (inference/kernels/transformerKernels_int8.cc.cu:1395-1499).  The bias is added
// in float for both storage types, as the reference does here.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
arrange_decself_qkv_kernel(const int8_t* __restrict__ ori_qkv, const T* __restrict__ qkv_bias,
                           int8_t* __restrict__ new_q, int8_t* __restrict__ new_k,
                           int8_t* __restrict__ new_v, int head_num, int dim_per_head,
                           int max_step, int step_id, float dequant_scale, float quant_scale) {
#pragma clang fp contract(off)
  const int H = head_num * dim_per_head;
  const int row = blockIdx.x, part = blockIdx.y;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float val = (float)ori_qkv[((long)row * 3 + part) * H + i] * dequant_scale +
                      TT<T>::ld(qkv_bias, (long)part * H + i);
    const int8_t qv = (int8_t)float2int8(val, quant_scale);
    if (part == 0) {
      new_q[(long)row * H + i] = qv;
    } else {
      const int head = i / dim_per_head, dim = i % dim_per_head;
      const long t = (((long)row * head_num + head) * max_step + step_id) * dim_per_head + dim;
      (part == 1 ? new_k : new_v)[t] = qv;
    }
  }
}

template <typename T>
int arrange_decself_qkv_i8I_i8O(int step_token_num, int hidden_size, hipStream_t s,
                                const int8_t* ori_qkv, const T* qkv_bias, int8_t* new_q,
                                int8_t* new_k, int8_t* new_v, int head_num, int dim_per_head,
                                int max_step, int step_id, float dequant_scale,
                                float quant_scale) {
  if (!ori_qkv || !qkv_bias || !new_q || !new_k || !new_v || step_token_num <= 0 ||
      head_num <= 0 || dim_per_head <= 0 || hidden_size != head_num * dim_per_head)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_decself_qkv_i8I_i8O: bad arguments");
  if (step_id < 0 || step_id >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_decself_qkv_i8I_i8O: step_id outside the cache");
  arrange_decself_qkv_kernel<T><<<dim3(step_token_num, 3), 256, 0, s>>>(
      ori_qkv, qkv_bias, new_q, new_k, new_v, head_num, dim_per_head, max_step, step_id,
      dequant_scale, quant_scale);
  return lsh_check_launch("arrange_decself_qkv_kernel");
}
template int arrange_decself_qkv_i8I_i8O<float>(int, int, hipStream_t, const int8_t*, const float*,
                                                int8_t*, int8_t*, int8_t*, int, int, int, int,
                                                float, float);
template int arrange_decself_qkv_i8I_i8O<__half>(int, int, hipStream_t, const int8_t*,
                                                 const __half*, int8_t*, int8_t*, int8_t*, int,
                                                 int, int, int, float, float);

// ---------------------------------------------------------------------------------
// decoder self attention over the int8 cache
//   scores[j]  = sum_d q[d] * K[j][d]                      (int32, exact)
//   val[j]     = float(scores[j]) * dq * dq * attn_scale
//   p[j]       = exp(val[j] - max) / sum
//   out[d]     = float2int8(sum_j float(V[j][d]) * p[j] * dq, quant_scale)
// (inference/model/quant_decoder.cc.cu:676-700 and
//  inference/kernels/transformerKernels_int8.cc.cu:1515-1594).
// One wavefront per (row, head); the value sum runs over j in ascending order.
// MODE 0: write the int32 scores only; 1: read scores, write new value; 2: fused.
// ---------------------------------------------------------------------------------
__device__ __forceinline__ int dot_i8_row(const int8_t* __restrict__ a,
                                          const int8_t* __restrict__ b, int d) {
  int acc = 0;
  if ((d & 3) == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 3) == 0) {
    const uint32_t* aw = reinterpret_cast<const uint32_t*>(a);
    const uint32_t* bw = reinterpret_cast<const uint32_t*>(b);
    for (int w = 0; w < (d >> 2); ++w) {
      const uint32_t x = aw[w], y = bw[w];
#pragma unroll
      for (int k = 0; k < 4; ++k) acc += unpack_i8(x, k) * unpack_i8(y, k);
    }
  } else {
    for (int k = 0; k < d; ++k) acc += (int)a[k] * (int)b[k];
  }
  return acc;
}

template <int MODE>
__global__ void __launch_bounds__(256)
decself_attn_kernel(int32_t* __restrict__ scores, const int8_t* __restrict__ q,
                    const int8_t* __restrict__ k_cache, const int8_t* __restrict__ v_cache,
                    int8_t* __restrict__ new_v, long bh_total, int step_num, int max_step,
                    int head_num, int d, float attn_scale, float dq, float quant_scale) {
#pragma clang fp contract(off)
  extern __shared__ float probs_all[];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const long bh = (long)blockIdx.x * 4 + wid;
  if (bh >= bh_total) return;  // whole wavefronts leave; no block barrier below
  const int padded = (step_num + 63) & ~63;
  float* probs = probs_all + (long)wid * padded;
  const int8_t* kb = k_cache + bh * (long)max_step * d;
  const int8_t* vb = v_cache + bh * (long)max_step * d;

  float mx = kFloatInfNeg;
  for (int j = lane; j < padded; j += 64) {
    float val = kFloatInfNeg;
    if (j < step_num) {
      int sc;
      if (MODE == 1) {
        sc = scores[bh * max_step + j];
      } else {
        sc = dot_i8_row(q + bh * d, kb + (long)j * d, d);
        if (MODE == 0) scores[bh * max_step + j] = sc;
      }
      val = (float)sc * dq * dq * attn_scale;
    }
    if (MODE != 0) probs[j] = val;
    mx = fmaxf(mx, val);
  }
  if (MODE == 0) return;
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j < padded; j += 64) {
    const float e = j < step_num ? __expf(probs[j] - mx) : 0.f;
    probs[j] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for (int j = lane; j < padded; j += 64) probs[j] = probs[j] / sum;
  // each lane re-reads values written by other lanes of its own wavefront
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const long row = bh / head_num;
  const int head = (int)(bh % head_num);
  for (int dd = lane; dd < d; dd += 64) {
    float acc = 0.f;
    for (int j = 0; j < step_num; ++j) acc += (float)vb[(long)j * d + dd] * probs[j] * dq;
    new_v[row * ((long)head_num * d) + (long)head * d + dd] = (int8_t)float2int8(acc, quant_scale);
  }
}

// The fused form at decode sizes: one workgroup (4 wavefronts) per (row, head).  A cached
// key or value row of d bytes is read by d/16 adjacent lanes with one 16-byte load each, so a
// wavefront covers 1024 contiguous bytes of cache per load instruction and every byte of
// the cache is read once.  Scores are exact int32 dot products (v_dot4), probabilities live
// in LDS, the value sum is accumulated per lane over its share of the steps and then reduced
// across lanes (shuffles) and wavefronts (LDS): a tree instead of the ascending-step order
// of the kernel above, so a context code can differ by one from it where the float sum
// lands next to a rounding boundary.  Requires d in {32, 64, 128} and 16-byte aligned rows.
template <int D, int NWV, int UN>
__global__ void __launch_bounds__(64 * NWV)
decself_attn_wg_kernel(const int8_t* __restrict__ q, const int8_t* __restrict__ k_cache,
                       const int8_t* __restrict__ v_cache, int8_t* __restrict__ new_v,
                       int step_num, int max_step, int head_num, float attn_scale, float dq,
                       float quant_scale) {
  extern __shared__ __align__(16) float lds_f[];
  // grid: x = head, y = row (no division before the first load)
  const int head = (int)blockIdx.x;
  const long row = blockIdx.y;
  const long bh = row * head_num + head;
  decself_attend_row<D, NWV, UN>(q + bh * D, k_cache + bh * (long)max_step * D,
                                 v_cache + bh * (long)max_step * D,
                                 new_v + row * ((long)head_num * D) + (long)head * D, true, step_num,
                                 attn_scale, dq, quant_scale, lds_f, threadIdx.x >> 6,
                                 threadIdx.x & 63);
}

// Short caches (one wavefront's loads cover them: at most 8 * 1024 / D steps): four (row, head)
// pairs per workgroup, one wavefront each, so that a step's attention is one round of the
// chip instead of four (1024 pairs at batch 16 x beam 4 x 16 heads).
template <int D, int UN>
__global__ void __launch_bounds__(256)
decself_attn_pack_kernel(const int8_t* __restrict__ q, const int8_t* __restrict__ k_cache,
                         const int8_t* __restrict__ v_cache, int8_t* __restrict__ new_v,
                         long bh_total, int step_num, int max_step, float attn_scale, float dq,
                         float quant_scale) {
  extern __shared__ __align__(16) float lds_f[];
  const int wave = threadIdx.x >> 6;
  const long bh_raw = (long)blockIdx.x * 4 + wave;
  const bool live = bh_raw < bh_total;
  const long bh = live ? bh_raw : bh_total - 1;
  // new_v is [rows, heads * D] and a pair's D codes sit at bh * D of it
  decself_attend_row_once<D, 1, UN>(q + bh * D, k_cache + bh * (long)max_step * D,
                                    v_cache + bh * (long)max_step * D, new_v + bh * D, live,
                                    step_num, attn_scale, dq, quant_scale,
                                    lds_f + wave * decself_group_floats<D, 1>(step_num), 0,
                                    threadIdx.x & 63);
}

static int decself_check(long bh_total, int step_num, int max_step, int head_num, int d) {
  if (bh_total <= 0 || head_num <= 0 || d <= 0 || max_step <= 0)
    return lsh_fail(LSH_ERR_INVALID, "decoder self attention: bad shape");
  if (step_num <= 0 || step_num > max_step)
    return lsh_fail(LSH_ERR_INVALID, "decoder self attention: step_num outside the cache");
  if (max_step > 4096)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "decoder self attention: max_step above 4096");
  return LSH_OK;
}

static size_t decself_lds(int step_num) { return (size_t)4 * ((step_num + 63) & ~63) * sizeof(float); }

int decself_scores_i8(const int8_t* q, const int8_t* k_cache, int32_t* scores, int batch_head_num,
                      int step_num, int max_step, int dim_per_head, hipStream_t s) {
  if (!q || !k_cache || !scores) return lsh_fail(LSH_ERR_INVALID, "decself_scores: null pointer");
  if (int rc = decself_check(batch_head_num, step_num, max_step, 1, dim_per_head)) return rc;
  decself_attn_kernel<0><<<(batch_head_num + 3) / 4, 256, 0, s>>>(
      scores, q, k_cache, nullptr, nullptr, batch_head_num, step_num, max_step, 1, dim_per_head,
      0.f, 0.f, 0.f);
  return lsh_check_launch("decself_attn_kernel<0>");
}

int fuse_softmax_new_value_i32I_i8O(const int32_t* correlation, const int8_t* v, int8_t* new_v,
                                    int batch_head_num, int step_num, int max_step, int head_num,
                                    int dim_per_head, float attn_scale, float dequant_scale,
                                    float quant_scale, hipStream_t s) {
  if (!correlation || !v || !new_v)
    return lsh_fail(LSH_ERR_INVALID, "ker_fuse_softmax_new_value_i32I_i8O: null pointer");
  if (int rc = decself_check(batch_head_num, step_num, max_step, head_num, dim_per_head)) return rc;
  decself_attn_kernel<1><<<(batch_head_num + 3) / 4, 256, decself_lds(step_num), s>>>(
      const_cast<int32_t*>(correlation), nullptr, nullptr, v, new_v, batch_head_num, step_num,
      max_step, head_num, dim_per_head, attn_scale, dequant_scale, quant_scale);
  return lsh_check_launch("decself_attn_kernel<1>");
}

int decself_attention_i8(const int8_t* q, const int8_t* k_cache, const int8_t* v_cache,
                         int8_t* new_v, int batch_head_num, int step_num, int max_step,
                         int head_num, int dim_per_head, float attn_scale, float dequant_scale,
                         float quant_scale, hipStream_t s) {
  if (!q || !k_cache || !v_cache || !new_v)
    return lsh_fail(LSH_ERR_INVALID, "decself_attention: null pointer");
  if (int rc = decself_check(batch_head_num, step_num, max_step, head_num, dim_per_head)) return rc;
  const bool aligned = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_cache) |
                         reinterpret_cast<uintptr_t>(v_cache)) & 15u) == 0;
  if (aligned && batch_head_num % head_num == 0 && batch_head_num / head_num <= 65535 &&
      (dim_per_head == 32 || dim_per_head == 64 || dim_per_head == 128)) {
    // 8 wavefronts per (row, head) once the cache is long (width buys loads in flight), 4
    // below, 1 (four pairs per workgroup) where one wavefront's loads cover the cache.  The
    // choice depends on the step count only, never on the number of rows: the widths sum the
    // values in different trees, and a row's result must not depend on its batch.  The loads
    // in flight per lane (UN) follow the cache length too: unrolled rounds that a short cache
    // never fills are code to fetch and clamped loads to wait for.
    const bool wide = step_num > 256;
    const dim3 grid(head_num, batch_head_num / head_num);
    const int kpw = 1024 / dim_per_head;  // cached steps per load instruction of a wavefront
    if (step_num <= 8 * kpw) {
#define LSH_DECSELF_PACK(D)                                                                      \
  if (step_num <= 4 * kpw)                                                                       \
    decself_attn_pack_kernel<D, 4>                                                               \
        <<<(batch_head_num + 3) / 4, 256, 4 * decself_group_floats<D, 1>(step_num) * sizeof(float), \
           s>>>(q, k_cache, v_cache, new_v, batch_head_num, step_num, max_step, attn_scale,      \
                dequant_scale, quant_scale);                                                     \
  else                                                                                           \
    decself_attn_pack_kernel<D, 8>                                                               \
        <<<(batch_head_num + 3) / 4, 256, 4 * decself_group_floats<D, 1>(step_num) * sizeof(float), \
           s>>>(q, k_cache, v_cache, new_v, batch_head_num, step_num, max_step, attn_scale,      \
                dequant_scale, quant_scale)
      if (dim_per_head == 32) { LSH_DECSELF_PACK(32); }
      else if (dim_per_head == 64) { LSH_DECSELF_PACK(64); }
      else { LSH_DECSELF_PACK(128); }
#undef LSH_DECSELF_PACK
      return lsh_check_launch("decself_attn_pack_kernel");
    }
    // loads per lane of the 8-wavefront form: as many as the cache needs (a slot beyond the cache
    // is a clamped load and a dead row of arithmetic; the lanes' rows and the order of their
    // sums do not depend on it, so neither do the bits)
    const int un8 = (step_num + 8 * kpw - 1) / (8 * kpw);
#define LSH_DECSELF_WIDE(D, UN)                                                                 \
  decself_attn_wg_kernel<D, 8, UN>                                                              \
      <<<grid, 512, decself_group_floats<D, 8>(step_num) * sizeof(float), s>>>(                 \
          q, k_cache, v_cache, new_v, step_num, max_step, head_num, attn_scale, dequant_scale,  \
          quant_scale)
#define LSH_DECSELF(D)                                                                          \
  if (wide) {                                                                                   \
    if (un8 <= 3) LSH_DECSELF_WIDE(D, 3);                                                       \
    else if (un8 == 4) LSH_DECSELF_WIDE(D, 4);                                                  \
    else if (un8 == 5) LSH_DECSELF_WIDE(D, 5);                                                  \
    else if (un8 == 6) LSH_DECSELF_WIDE(D, 6);                                                  \
    else LSH_DECSELF_WIDE(D, 8);                                                                \
  } else /* 8192 / D < step_num <= 256 */                                                         \
    decself_attn_wg_kernel<D, 4, 4>                                                             \
        <<<grid, 256, decself_group_floats<D, 4>(step_num) * sizeof(float), s>>>(               \
        q, k_cache, v_cache, new_v, step_num, max_step, head_num, attn_scale, dequant_scale,    \
        quant_scale)
    if (dim_per_head == 32) { LSH_DECSELF(32); }
    else if (dim_per_head == 64) { LSH_DECSELF(64); }
    else { LSH_DECSELF(128); }
#undef LSH_DECSELF
#undef LSH_DECSELF_WIDE
    return lsh_check_launch("decself_attn_wg_kernel");
  }
  decself_attn_kernel<2><<<(batch_head_num + 3) / 4, 256, decself_lds(step_num), s>>>(
      nullptr, q, k_cache, v_cache, new_v, batch_head_num, step_num, max_step, head_num,
      dim_per_head, attn_scale, dequant_scale, quant_scale);
  return lsh_check_launch("decself_attn_kernel<2>");
}

// ---------------------------------------------------------------------------------
// encoder-decoder attention: query re-layout
// (inference/kernels/transformerKernels_int8.cc.cu:1596-1688)
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
arrange_encdec_q_kernel(const int8_t* __restrict__ ori_q, const T* __restrict__ q_bias,
                        T* __restrict__ new_q, int beam_size, int dim_per_head, int head_num,
                        float dequant_scale) {
#pragma clang fp contract(off)
  const int H = dim_per_head * head_num;
  const int row = blockIdx.x;
  const int batch_id = row / beam_size, beam_id = row % beam_size;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    // fp16: half(code * dq) + bias as a half add; fp32: plain float arithmetic
    const int code = ori_q[(long)row * H + i];
    const float bias = TT<T>::ld(q_bias, i);
    const float val = TT<T>::is_half ? dequant_add_bias_h(code, dequant_scale, bias)
                                     : (float)code * dequant_scale + bias;
    const int head = i / dim_per_head, dim = i % dim_per_head;
    TT<T>::st(new_q,
              (((long)batch_id * head_num + head) * beam_size + beam_id) * dim_per_head + dim, val);
  }
}

template <typename T>
int arrange_encdec_q_i8I(int step_token_num, int hidden_size, hipStream_t s, const int8_t* ori_q,
                         const T* q_bias, T* new_q, int beam_size, int dim_per_head, int head_num,
                         float dequant_scale) {
  if (!ori_q || !q_bias || !new_q || step_token_num <= 0 || beam_size <= 0 ||
      step_token_num % beam_size != 0 || hidden_size != dim_per_head * head_num)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_encdec_q_i8I: bad arguments");
  arrange_encdec_q_kernel<T><<<step_token_num, 256, 0, s>>>(ori_q, q_bias, new_q, beam_size,
                                                            dim_per_head, head_num, dequant_scale);
  return lsh_check_launch("arrange_encdec_q_kernel");
}
template int arrange_encdec_q_i8I<float>(int, int, hipStream_t, const int8_t*, const float*, float*,
                                         int, int, int, float);
template int arrange_encdec_q_i8I<__half>(int, int, hipStream_t, const int8_t*, const __half*,
                                          __half*, int, int, int, float);

// ---------------------------------------------------------------------------------
// projected encoder output -> per-layer K and V in [batch, head, seq, dim]
// (inference/kernels/transformerKernels.cc.cu:903-1020)
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
arrange_encdec_kv_kernel(const T* __restrict__ ori_kv, const T* __restrict__ kv_bias,
                         T* __restrict__ new_k, T* __restrict__ new_v, long offset_per_layer,
                         int batch_seq_len, int dim_per_head, int head_num) {
  const int H = dim_per_head * head_num;
  const long tok = blockIdx.x;
  const int y = blockIdx.y;
  const long seq_id = tok / batch_seq_len, token_id = tok % batch_seq_len;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float val = TT<T>::ld(ori_kv, (tok * gridDim.y + y) * H + i) +
                      TT<T>::ld(kv_bias, (long)y * H + i);  // rounded to T by the store
    const int head = i / dim_per_head, dim = i % dim_per_head;
    const long t = ((seq_id * head_num + head) * batch_seq_len + token_id) * dim_per_head + dim +
                   (long)(y >> 1) * offset_per_layer;
    TT<T>::st((y & 1) ? new_v : new_k, t, val);
  }
}

template <typename T>
int arrange_encdec_kv(int batch_token_num, int dec_layer_num, int hidden_size, hipStream_t s,
                      const T* ori_kv, const T* kv_bias, T* new_k, T* new_v,
                      long offset_per_layer, int batch_seq_len, int dim_per_head, int head_num) {
  if (!ori_kv || !kv_bias || !new_k || !new_v || batch_token_num <= 0 || dec_layer_num <= 0 ||
      batch_seq_len <= 0 || batch_token_num % batch_seq_len != 0 ||
      hidden_size != dim_per_head * head_num)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_encdec_kv: bad arguments");
  if (dec_layer_num * 2 > 65535)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "ker_arrange_encdec_kv: too many layers");
  if (offset_per_layer < (long)batch_token_num * hidden_size)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_encdec_kv: layers would overlap");
  arrange_encdec_kv_kernel<T><<<dim3(batch_token_num, dec_layer_num * 2), 256, 0, s>>>(
      ori_kv, kv_bias, new_k, new_v, offset_per_layer, batch_seq_len, dim_per_head, head_num);
  return lsh_check_launch("arrange_encdec_kv_kernel");
}
template int arrange_encdec_kv<float>(int, int, int, hipStream_t, const float*, const float*,
                                      float*, float*, long, int, int, int);
template int arrange_encdec_kv<__half>(int, int, int, hipStream_t, const __half*, const __half*,
                                       __half*, __half*, long, int, int, int);

// ---------------------------------------------------------------------------------
// softmax of the encoder-decoder correlation, keys masked by the source padding
// (inference/kernels/transformerKernels.cc.cu:1226-1284); one wavefront per row
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
softmax_encdec_kernel(T* corr, const int* __restrict__ pad_mask, long rows, int rows_per_batch,
                      int seq_len) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int* mask = pad_mask + (row / rows_per_batch) * seq_len;
  T* p = corr + row * seq_len;
  float mx = kFloatInfNeg;
  for (int j = lane; j < seq_len; j += 64)
    if (!mask[j]) mx = fmaxf(mx, TT<T>::ld(p, j));
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j < seq_len; j += 64)
    if (!mask[j]) sum += __expf(TT<T>::ld(p, j) - mx);
  sum = wave_sum(sum);
  for (int j = lane; j < seq_len; j += 64) {
    const float e = mask[j] ? 0.f : __expf(TT<T>::ld(p, j) - mx);
    TT<T>::st(p, j, e / sum);
  }
}

template <typename T>
int correlation_softmax_encdec(int batch_size, int head_num_per_seq, int batch_seq_len,
                               hipStream_t s, T* correlation, const int* src_padding_mask) {
  if (!correlation || !src_padding_mask || batch_size <= 0 || head_num_per_seq <= 0 ||
      batch_seq_len <= 0)
    return lsh_fail(LSH_ERR_INVALID, "ker_correlation_softmax_encdec: bad arguments");
  const long rows = (long)batch_size * head_num_per_seq;
  softmax_encdec_kernel<T><<<(int)((rows + 3) / 4), 256, 0, s>>>(
      correlation, src_padding_mask, rows, head_num_per_seq, batch_seq_len);
  return lsh_check_launch("softmax_encdec_kernel");
}
template int correlation_softmax_encdec<float>(int, int, int, hipStream_t, float*, const int*);
template int correlation_softmax_encdec<__half>(int, int, int, hipStream_t, __half*, const int*);

// ---------------------------------------------------------------------------------
// Fused encoder-decoder attention (fp16), one wavefront per (batch, head, beam):
//   s[j] = half(half(1/sqrt(d)) * sum_d q[d] k[j][d]);  p = half(masked softmax(s));
//   c[d] = half(sum_j p[j] v[j][d]);  out = float2int8(c, quant_scale) in [rows, H]
// i.e. the two strided-batched GEMMs, ker_correlation_softmax_encdec and
// ker_arrange_atten_output_i8O of inference/model/quant_decoder.cc.cu:765-800 with
// their fp16 rounding points kept.
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
encdec_attn_kernel(const __half* __restrict__ q, const __half* __restrict__ k,
                   const __half* __restrict__ v, const int* __restrict__ pad_mask,
                   __half* __restrict__ ctx, int8_t* __restrict__ ctx_q, float quant_scale,
                   long waves_total, int beam_size, int head_num, int seq_len, int d,
                   float alpha_h) {
#pragma clang fp contract(off)
  extern __shared__ float probs_all[];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const long w = (long)blockIdx.x * 4 + wid;
  if (w >= waves_total) return;
  const int padded = (seq_len + 63) & ~63;
  float* probs = probs_all + (long)wid * padded;
  const long bh = w / beam_size;
  const int beam = (int)(w % beam_size);
  const long b = bh / head_num;
  const int head = (int)(bh % head_num);
  const int* mask = pad_mask + b * seq_len;
  const __half* qp = q + w * d;  // [B, h, beam, d]
  const __half* kb = k + bh * (long)seq_len * d;
  const __half* vb = v + bh * (long)seq_len * d;

  float mx = kFloatInfNeg;
  for (int j = lane; j < padded; j += 64) {
    float sc = kFloatInfNeg;
    if (j < seq_len) {
      float acc = 0.f;
      const __half* kr = kb + (long)j * d;
      for (int dd = 0; dd < d; ++dd) acc += __half2float(qp[dd]) * __half2float(kr[dd]);
      sc = TT<__half>::rnd(alpha_h * acc);
      if (!mask[j]) mx = fmaxf(mx, sc);
    }
    probs[j] = sc;
  }
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j < padded; j += 64) {
    const float e = (j < seq_len && !mask[j]) ? __expf(probs[j] - mx) : 0.f;
    probs[j] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for (int j = lane; j < padded; j += 64) probs[j] = TT<__half>::rnd(probs[j] / sum);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const long row = b * beam_size + beam;
  for (int dd = lane; dd < d; dd += 64) {
    float acc = 0.f;
    for (int j = 0; j < seq_len; ++j) acc += probs[j] * __half2float(vb[(long)j * d + dd]);
    const float c = TT<__half>::rnd(acc);
    if (ctx) ctx[w * d + dd] = __float2half_rn(c);
    if (ctx_q)
      ctx_q[row * ((long)head_num * d) + (long)head * d + dd] = (int8_t)float2int8(c, quant_scale);
  }
}

// The same for head sizes 32 / 64 / 128 with 16-byte aligned operands: a key row and the
// query are read as 16-byte vectors and the value rows eight steps at a time, every load
// issued before the first is used; the sums run in the same order as above (dimension by
// dimension for a score, step by step for a context element), so the results are the same
// bits.
template <int D>
__global__ void __launch_bounds__(256)
encdec_attn_vec_kernel(const __half* __restrict__ q, const __half* __restrict__ k,
                       const __half* __restrict__ v, const int* __restrict__ pad_mask,
                       __half* __restrict__ ctx, int8_t* __restrict__ ctx_q, float quant_scale,
                       long waves_total, int beam_size, int head_num, int seq_len,
                       float alpha_h) {
#pragma clang fp contract(off)
  extern __shared__ float probs_all[];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const long w = (long)blockIdx.x * 4 + wid;
  if (w >= waves_total) return;
  const int padded = (seq_len + 63) & ~63;
  float* probs = probs_all + (long)wid * padded;
  const long bh = w / beam_size;
  const int beam = (int)(w % beam_size);
  const long b = bh / head_num;
  const int head = (int)(bh % head_num);
  const int* mask = pad_mask + b * seq_len;
  const __half* qp = q + w * D;  // [B, h, beam, d]
  const __half* kb = k + bh * (long)seq_len * D;
  const __half* vb = v + bh * (long)seq_len * D;

  half8_t qv[D / 8];
#pragma unroll
  for (int c = 0; c < D / 8; ++c) qv[c] = *reinterpret_cast<const half8_t*>(qp + c * 8);

  float mx = kFloatInfNeg;
  for (int j = lane; j < padded; j += 64) {
    float sc = kFloatInfNeg;
    if (j < seq_len) {
      half8_t kv[D / 8];
#pragma unroll
      for (int c = 0; c < D / 8; ++c)
        kv[c] = *reinterpret_cast<const half8_t*>(kb + (long)j * D + c * 8);
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < D / 8; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += __half2float(qv[c].v[e]) * __half2float(kv[c].v[e]);
      sc = TT<__half>::rnd(alpha_h * acc);
      if (!mask[j]) mx = fmaxf(mx, sc);
    }
    probs[j] = sc;
  }
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j < padded; j += 64) {
    const float e = (j < seq_len && !mask[j]) ? __expf(probs[j] - mx) : 0.f;
    probs[j] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for (int j = lane; j < padded; j += 64) probs[j] = TT<__half>::rnd(probs[j] / sum);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const long row = b * beam_size + beam;
  for (int dd = lane; dd < D; dd += 64) {
    float acc = 0.f;
    constexpr int UV = 32;  // value rows in flight per lane
    for (int j0 = 0; j0 < seq_len; j0 += UV) {
      __half vv[UV];
#pragma unroll
      for (int u = 0; u < UV; ++u)  // clamped, not predicated: the loads stay back to back
        vv[u] = vb[(long)min(j0 + u, seq_len - 1) * D + dd];
#pragma unroll
      for (int u = 0; u < UV; ++u)
        if (j0 + u < seq_len) acc += probs[j0 + u] * __half2float(vv[u]);
    }
    const float c = TT<__half>::rnd(acc);
    if (ctx) ctx[w * D + dd] = __float2half_rn(c);
    if (ctx_q)
      ctx_q[row * ((long)head_num * D) + (long)head * D + dd] = (int8_t)float2int8(c, quant_scale);
  }
}

// Short sources (at most 16 loads of a wavefront cover the keys): one wavefront per (sentence,
// head, beam) as above, laid out for a generation step that lasts a few microseconds.  D / 8
// adjacent lanes share a key or value row (16-byte loads, a load instruction of the wavefront
// reads whole rows back to back), keys and values are requested together before anything is
// used, scores and probabilities stay in the registers of the lanes that use them, the sums
// over lanes are DPP permutations and lane reads, and only the D partial context sums of the
// wavefront's four rows of 16 lanes meet in LDS.  The rounding points are those of the
// kernels above (score, probability and context element rounded to fp16); the sums run in
// another order.
//
// QPROD: the query is not read but made here, by the product that precedes the attention in a
// decoder layer (x int8 [rows, hidden] times the head's D rows of W [hidden, hidden], the
// epilogue of gemm_i8_encdec_q_f16: the same fp16 values).  D = 64, at most 4 beams, hidden a
// multiple of 64 up to 1024, eight wavefronts: wavefront 4 + w multiplies columns 16 w ..
// 16 w + 15 of the head for the sentence's beams (v_mfma_i32_16x16x64_i8, weights as the row
// operand, fragments straight from memory) and leaves the values in LDS, while wavefront b
// requests the keys, values and mask of beam b; after the barrier the product wavefronts are
// done and wavefront b goes on with beam b.  Two short instruction streams side by side
// instead of one long one, and the two memory streams travel together.
struct EncdecQProd {
  const int8_t* x;
  const int8_t* W;
  const __half* bias;
  int hidden;
  float alpha, dequant_scale;
};

template <int D, int UN, bool QPROD = false>
__global__ void __launch_bounds__(QPROD ? 512 : 256)
encdec_attn_short_kernel(const __half* __restrict__ q, const __half* __restrict__ k,
                         const __half* __restrict__ v, const int* __restrict__ pad_mask,
                         __half* __restrict__ ctx, int8_t* __restrict__ ctx_q, float quant_scale,
                         int beam_size, int head_num, int seq_len, float alpha_h,
                         EncdecQProd qp = EncdecQProd{}) {
#pragma clang fp contract(off)
  constexpr int CH = D / 8;     // lanes per row
  constexpr int KPW = 64 / CH;  // rows per load instruction of the wavefront
  __shared__ float part_all[4][4][D];
  __shared__ __align__(16) __half q_lds[QPROD ? 4 * D : 8];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  // grid: x = head, y = sentence, z = groups of 4 beams; wavefront = beam
  const int head = (int)blockIdx.x, beam = (int)blockIdx.z * 4 + wid;
  const long b = blockIdx.y;
  const bool alive = beam < beam_size;
  const int bm = alive ? beam : beam_size - 1;
  const long bh = b * head_num + head;
  const long w = bh * beam_size + bm;
  const int c = lane % CH, grp = lane / CH;
  const int* mask = pad_mask + b * seq_len;
  const __half* kb = k + bh * (long)seq_len * D + c * 8;
  const __half* vb = v + bh * (long)seq_len * D + c * 8;
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  union Row {
    uint4 u;
    h2 p[4];
    __half h[8];
  };
  if constexpr (QPROD) {
    if (wid >= 4) {  // the product wavefronts
      const int pw = wid - 4;
      typedef int v4i __attribute__((ext_vector_type(4)));
      const int KS = qp.hidden >> 6;  // 64-byte K slices (<= 16)
      const int m = lane & 15, kq = lane >> 4;
      // matrix row m: beam m of the sentence (rows beyond the beams repeat the last one)
      const int8_t* xp = qp.x + (b * beam_size + min(m, beam_size - 1)) * (long)qp.hidden + kq * 16;
      // the row operand: column 16 pw + m of the head
      const int8_t* wp = qp.W + ((long)head * D + pw * 16 + m) * (long)qp.hidden + kq * 16;
      const uint2 braw = *reinterpret_cast<const uint2*>(qp.bias + head * D + pw * 16 + 4 * kq);
      v4i xf[16], wf[16];
#pragma unroll
      for (int sl = 0; sl < 16; ++sl) wf[sl] = *reinterpret_cast<const v4i*>(wp + min(sl, KS - 1) * 64);
#pragma unroll
      for (int sl = 0; sl < 16; ++sl) xf[sl] = *reinterpret_cast<const v4i*>(xp + min(sl, KS - 1) * 64);
      __builtin_amdgcn_sched_barrier(0);  // every request of the kernel is out before a product
      v4i acc = (v4i)0;
#pragma unroll
      for (int sl = 0; sl < 16; ++sl) {
        asm volatile("" : "+v"(wf[sl]));
        asm volatile("" : "+v"(xf[sl]));
        if (sl < KS) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[sl], xf[sl], acc, 0, 0, 0);
      }
      // lane holds the product of beam m with columns 16 pw + 4 kq + 0..3 of the head
      if (m < beam_size) {
        union {
          uint2 u;
          __half h[4];
        } bb, out;
        bb.u = braw;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          out.h[i] = __float2half_rn(dequant_add_bias_h(requant_acc(acc[i], qp.alpha),
                                                        qp.dequant_scale, __half2float(bb.h[i])));
        *reinterpret_cast<uint2*>(q_lds + m * D + pw * 16 + 4 * kq) = out.u;
      }
      __syncthreads();
      return;
    }
  }
  Row qv, kv[UN], vv[UN];
  int mk[UN];
  if (!QPROD) qv.u = *reinterpret_cast<const uint4*>(q + w * D + c * 8);
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const int j = min(u * KPW + grp, seq_len - 1);  // clamped, not predicated
    kv[u].u = *reinterpret_cast<const uint4*>(kb + (long)j * D);
    mk[u] = mask[j];
  }
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const int j = min(u * KPW + grp, seq_len - 1);
    vv[u].u = *reinterpret_cast<const uint4*>(vb + (long)j * D);
  }
  if constexpr (QPROD) {
    __syncthreads();
    qv.u = *reinterpret_cast<const uint4*>(q_lds + bm * D + c * 8);
  }
  // every load is requested before the first product: left alone the scheduler moves half of
  // the value loads behind the soft-max, a second trip to memory in a kernel of one
  __builtin_amdgcn_sched_barrier(0);
  float val[UN];
  float mx = kFloatInfNeg;
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_fdot2(qv.p[e], kv[u].p[e], acc, false);
    // the CH partial dot products of the row
    acc += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, acc), 0xB1, 0xf, 0xf, false));
    acc += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, acc), 0x4E, 0xf, 0xf, false));
    if (CH >= 8)
      acc += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, acc), 0x141, 0xf, 0xf, false));
    if (CH >= 16)
      acc += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, acc), 0x140, 0xf, 0xf, false));
    const bool valid = u * KPW + grp < seq_len && !mk[u];
    val[u] = TT<__half>::rnd(alpha_h * acc);
    if (valid) mx = fmaxf(mx, val[u]);
    else val[u] = kFloatInfNeg;
  }
  mx = row_ror_max<8>(row_ror_max<4>(row_ror_max<2>(row_ror_max<1>(mx))));
  mx = fmaxf(fmaxf(lane_of(mx, 0), lane_of(mx, 16)), fmaxf(lane_of(mx, 32), lane_of(mx, 48)));
  float sum = 0.f;
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    val[u] = val[u] > kFloatInfNeg ? __expf(val[u] - mx) : 0.f;
    sum += val[u];
  }
  // every row once: lanes of one c, rotations by multiples of CH within a row of 16 lanes
  if (CH <= 4) sum = row_ror_add<4>(sum);
  if (CH <= 8) sum = row_ror_add<8>(sum);
  sum = (lane_of(sum, 0) + lane_of(sum, 16)) + (lane_of(sum, 32) + lane_of(sum, 48));
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const float p = TT<__half>::rnd(val[u] / sum);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(p, __half2float(vv[u].h[e]), acc[e]);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if (CH <= 4) acc[e] = row_ror_add<4>(acc[e]);
    if (CH <= 8) acc[e] = row_ror_add<8>(acc[e]);
  }
  float* part = &part_all[wid][0][0];
  if ((lane & 15) < CH) {
    float* pp = part + (lane >> 4) * D + c * 8;
    *reinterpret_cast<float4*>(pp) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    *reinterpret_cast<float4*>(pp + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (!alive) return;
  const long row = b * beam_size + beam;
  for (int dd = lane; dd < D; dd += 64) {
    const float t = (part[dd] + part[D + dd]) + (part[2 * D + dd] + part[3 * D + dd]);
    const float cv = TT<__half>::rnd(t);
    if (ctx) ctx[w * D + dd] = __float2half_rn(cv);
    if (ctx_q)
      ctx_q[row * ((long)head_num * D) + (long)head * D + dd] = (int8_t)float2int8(cv, quant_scale);
  }
}

// The query product of a decoder layer and its cross attention as one launch, where the short
// kernel covers the shape: the fp16 query never leaves the compute unit.  ctx_q must not
// overlap x (other workgroups still read the rows).
bool encdec_q_attention_supported(int beam_size, int head_num, int hidden, int batch_seq_len) {
  return beam_size >= 1 && beam_size <= 4 && head_num > 0 && hidden == head_num * 64 &&
         hidden <= 1024 && batch_seq_len >= 1 && batch_seq_len <= 16 * 8;
}

int encdec_q_attention_f16(const int8_t* x, const int8_t* q_weight, const __half* q_bias,
                           const __half* k, const __half* v, const int* pad_mask, int8_t* ctx_q,
                           float quant_scale, int batch_size, int beam_size, int head_num,
                           int batch_seq_len, int hidden, float alpha, float dequant_scale,
                           hipStream_t s) {
  if (!x || !q_weight || !q_bias || !k || !v || !pad_mask || !ctx_q || batch_size <= 0)
    return lsh_fail(LSH_ERR_INVALID, "encdec_q_attention: bad arguments");
  if (!encdec_q_attention_supported(beam_size, head_num, hidden, batch_seq_len) ||
      batch_size > 65535 ||
      ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(q_weight) |
        reinterpret_cast<uintptr_t>(q_bias) | reinterpret_cast<uintptr_t>(k) |
        reinterpret_cast<uintptr_t>(v)) & 15u) != 0)
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "encdec_q_attention: needs heads of 64, hidden <= 1024, at most 4 beams, a "
                    "source of at most 128 tokens, 16-byte aligned operands");
  const long rows = (long)batch_size * beam_size;
  if (x < ctx_q + rows * hidden && ctx_q < x + rows * hidden)
    return lsh_fail(LSH_ERR_INVALID, "encdec_q_attention: ctx_q overlaps x");
  const float alpha_h = __half2float(__float2half_rn(sqrtf(1.f / 64.f)));
  const dim3 grid(head_num, batch_size, 1);
  const EncdecQProd qp{x, q_weight, q_bias, hidden, alpha, dequant_scale};
  const int un = (batch_seq_len + 7) / 8;
#define LSH_ENCDEC_Q(UN)                                                                     \
  encdec_attn_short_kernel<64, UN, true><<<grid, 512, 0, s>>>(                               \
      nullptr, k, v, pad_mask, nullptr, ctx_q, quant_scale, beam_size, head_num, batch_seq_len, \
      alpha_h, qp)
  if (un <= 4) LSH_ENCDEC_Q(4);
  else if (un <= 8) LSH_ENCDEC_Q(8);
  else LSH_ENCDEC_Q(16);
#undef LSH_ENCDEC_Q
  return lsh_check_launch("encdec_attn_short_kernel<q product>");
}

int encdec_attention_f16(const __half* q, const __half* k, const __half* v, const int* pad_mask,
                         __half* ctx, int8_t* ctx_q, float quant_scale, int batch_size,
                         int beam_size, int head_num, int batch_seq_len, int dim_per_head,
                         hipStream_t s) {
  if (!q || !k || !v || !pad_mask || (!ctx && !ctx_q) || batch_size <= 0 || beam_size <= 0 ||
      head_num <= 0 || batch_seq_len <= 0 || dim_per_head <= 0)
    return lsh_fail(LSH_ERR_INVALID, "encdec_attention: bad arguments");
  if (batch_seq_len > 4096)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "encdec_attention: source length above 4096");
  const long waves = (long)batch_size * head_num * beam_size;
  const float alpha_h = __half2float(__float2half_rn(sqrtf(1.f / (float)dim_per_head)));
  const size_t lds = (size_t)4 * ((batch_seq_len + 63) & ~63) * sizeof(float);
  const bool aligned = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
                         reinterpret_cast<uintptr_t>(v)) & 15u) == 0;
  if (aligned && batch_size <= 65535 && beam_size <= 4 * 65535 &&
      (dim_per_head == 32 || dim_per_head == 64 || dim_per_head == 128) &&
      batch_seq_len <= 16 * (512 / dim_per_head)) {
    // short sources: keys, values and probabilities in registers.  The choice follows the
    // source length and the head size only, never the number of rows.
    const dim3 grid(head_num, batch_size, (beam_size + 3) / 4);
    const int kpw = 512 / dim_per_head;  // rows per load instruction of a wavefront
    const int un = (batch_seq_len + kpw - 1) / kpw;
#define LSH_ENCDEC_SHORT(D, UN)                                                                   \
  encdec_attn_short_kernel<D, UN><<<grid, 256, 0, s>>>(q, k, v, pad_mask, ctx, ctx_q, quant_scale, \
                                                       beam_size, head_num, batch_seq_len, alpha_h)
#define LSH_ENCDEC_SHORT_D(D)                \
  if (un <= 4) LSH_ENCDEC_SHORT(D, 4);       \
  else if (un <= 8) LSH_ENCDEC_SHORT(D, 8);  \
  else LSH_ENCDEC_SHORT(D, 16)
    if (dim_per_head == 32) { LSH_ENCDEC_SHORT_D(32); }
    else if (dim_per_head == 64) { LSH_ENCDEC_SHORT_D(64); }
    else { LSH_ENCDEC_SHORT_D(128); }
#undef LSH_ENCDEC_SHORT_D
#undef LSH_ENCDEC_SHORT
    return lsh_check_launch("encdec_attn_short_kernel");
  }
  if (aligned && (dim_per_head == 32 || dim_per_head == 64 || dim_per_head == 128)) {
#define LSH_ENCDEC(D)                                                                           \
  encdec_attn_vec_kernel<D><<<(int)((waves + 3) / 4), 256, lds, s>>>(                           \
      q, k, v, pad_mask, ctx, ctx_q, quant_scale, waves, beam_size, head_num, batch_seq_len,    \
      alpha_h)
    if (dim_per_head == 32) LSH_ENCDEC(32);
    else if (dim_per_head == 64) LSH_ENCDEC(64);
    else LSH_ENCDEC(128);
#undef LSH_ENCDEC
    return lsh_check_launch("encdec_attn_vec_kernel");
  }
  encdec_attn_kernel<<<(int)((waves + 3) / 4), 256, lds, s>>>(
      q, k, v, pad_mask, ctx, ctx_q, quant_scale, waves, beam_size, head_num, batch_seq_len,
      dim_per_head, alpha_h);
  return lsh_check_launch("encdec_attn_kernel");
}

}  // namespace lsh
