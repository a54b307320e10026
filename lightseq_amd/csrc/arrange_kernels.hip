// Head split / merge around the attention core and the int8-table embedding.
// Pure data movement with a dequant or quant on the way: 8 consecutive elements
// (one head-dim run) per thread, 8-byte int8 and 16-byte fp16 accesses.
//
// Replaces inference/kernels/transformerKernels_int8.cc.cu:1080-1393 and
// inference/kernels/embKernels_int8.cc.cu:13-155.
#include "ls_device.h"
#include "ls_launch.h"

#include <type_traits>

namespace lsh {

__device__ __forceinline__ void unpack8(uint2 w, float (&o)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    o[k] = (float)unpack_i8(w.x, k);
    o[4 + k] = (float)unpack_i8(w.y, k);
  }
}
__device__ __forceinline__ void ld8(const float* p, long i, float (&o)[8]) {
  float a[4], b[4];
  ld4(p, i, a);
  ld4(p, i + 4, b);
#pragma unroll
  for (int k = 0; k < 4; ++k) { o[k] = a[k]; o[4 + k] = b[k]; }
}
__device__ __forceinline__ void ld8(const __half* p, long i, float (&o)[8]) {
  half8_t t = *reinterpret_cast<const half8_t*>(p + i);
#pragma unroll
  for (int k = 0; k < 8; ++k) o[k] = __half2float(t.v[k]);
}
__device__ __forceinline__ void st8(float* p, long i, const float (&o)[8]) {
  *reinterpret_cast<float4*>(p + i) = make_float4(o[0], o[1], o[2], o[3]);
  *reinterpret_cast<float4*>(p + i + 4) = make_float4(o[4], o[5], o[6], o[7]);
}
__device__ __forceinline__ void st8(__half* p, long i, const float (&o)[8]) {
  half8_t t;
#pragma unroll
  for (int k = 0; k < 8; ++k) t.v[k] = __float2half_rn(o[k]);
  *reinterpret_cast<half8_t*>(p + i) = t;
}
__device__ __forceinline__ uint2 quant8(const float (&v)[8], float qs) {
  uint2 o;
  o.x = pack4_i8(float2int8(v[0], qs), float2int8(v[1], qs), float2int8(v[2], qs),
                 float2int8(v[3], qs));
  o.y = pack4_i8(float2int8(v[4], qs), float2int8(v[5], qs), float2int8(v[6], qs),
                 float2int8(v[7], qs));
  return o;
}

// ---------------------------------------------------------------------------------
// [M, 3, H] int8  ->  3 x [B, h, S, d] T      (V elements per thread, V in {8, 1})
// I8OUT: requantise q/k/v to int8 and also emit the dequantised v (GPT prefill).
template <typename T, int V, bool I8OUT>
__global__ void __launch_bounds__(256)
arrange_qkv_kernel(const int8_t* __restrict__ ori, const T* __restrict__ bias,
                   T* __restrict__ new_qkv, int8_t* __restrict__ q8, int8_t* __restrict__ k8,
                   int8_t* __restrict__ v8, T* __restrict__ d_v, long max_batch_dim, long total_v,
                   int seq_len, int d, int head_num, float ds, float qs) {
  const int hidden = d * head_num;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; idx < total_v; idx += stride) {
    const long e = idx * V;  // flat element index in [M, 3, H]
    const int i = (int)(e % hidden);
    const long tw = e / hidden;
    const int which = (int)(tw % 3);
    const long tok = tw / 3;
    const int b = (int)(tok / seq_len), s = (int)(tok % seq_len);
    const int head = i / d, dim = i % d;
    const long target = (((long)b * head_num + head) * seq_len + s) * d + dim;
    if (V == 8) {
      float x[8], bv[8];
      unpack8(*reinterpret_cast<const uint2*>(ori + e), x);
      ld8(bias, (long)which * hidden + i, bv);
      if (!I8OUT) {
        // fp16: T(x * ds) + bias as a half add; fp32: float add (rnd is the identity)
#pragma unroll
        for (int k = 0; k < 8; ++k)
          x[k] = TT<T>::is_half ? dequant_add_bias_h((int)x[k], ds, bv[k]) : x[k] * ds + bv[k];
        st8(new_qkv, max_batch_dim * which + target, x);
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) x[k] = x[k] * ds + bv[k];
        uint2 qv = quant8(x, qs);
        int8_t* dst = which == 0 ? q8 : (which == 1 ? k8 : v8);
        *reinterpret_cast<uint2*>(dst + target) = qv;
        if (which == 2) {
          float dv[8];
          unpack8(qv, dv);
#pragma unroll
          for (int k = 0; k < 8; ++k) dv[k] = dv[k] / qs;
          st8(d_v, target, dv);
        }
      }
    } else {
      float x = (float)ori[e] * ds;
      float bv = TT<T>::ld(bias, (long)which * hidden + i);
      if (!I8OUT) {
        TT<T>::st(new_qkv, max_batch_dim * which + target, TT<T>::rnd(x) + bv);
      } else {
        int qv = float2int8(x + bv, qs);
        int8_t* dst = which == 0 ? q8 : (which == 1 ? k8 : v8);
        dst[target] = (int8_t)qv;
        if (which == 2) TT<T>::st(d_v, target, (float)qv / qs);
      }
    }
  }
}

// The fp16 form for whole sequences: a workgroup owns one 128-byte column group (128 / d heads)
// of one part (q, k or v) of one sequence and walks its tokens, 32 rows per pass, 16 codes per
// thread.  What it writes is contiguous per head -- seq_len * d halfs -- instead of one
// 128-byte piece per head and token scattered over the three tensors, and the bias slice is
// loaded once.  Same arithmetic per element as the kernel above.
template <int UNR>
__global__ void __launch_bounds__(256)
arrange_qkv_heads_kernel(const int8_t* __restrict__ ori, const __half* __restrict__ bias,
                         __half* __restrict__ new_qkv, long max_batch_dim, int seq_len, int d,
                         int head_num, int groups, float ds) {
  const int hidden = d * head_num;
  const int grp = blockIdx.x % groups, which = (blockIdx.x / groups) % 3;
  const int b = blockIdx.x / (groups * 3);
  const int row = threadIdx.x >> 3, seg = threadIdx.x & 7;
  const int col = grp * 128 + seg * 16;  // first of this thread's 16 columns inside the part
  const int head = col / d, dim = col % d;
  float bv[16];
  {
    float lo[8], hi[8];
    ld8(bias, (long)which * hidden + col, lo);
    ld8(bias, (long)which * hidden + col + 8, hi);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      bv[k] = lo[k];
      bv[8 + k] = hi[k];
    }
  }
  const int8_t* src = ori + ((long)b * seq_len * 3 + which) * hidden + col;
  __half* dst = new_qkv + max_batch_dim * which + ((long)b * head_num + head) * seq_len * d + dim;
  for (int s0 = row; s0 < seq_len; s0 += 32 * UNR) {
    uint4 w[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int s = min(s0 + 32 * u, seq_len - 1);
      w[u] = *reinterpret_cast<const uint4*>(src + (long)s * 3 * hidden);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int s = s0 + 32 * u;
      if (s >= seq_len) break;
      const uint32_t wi[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
      float x[16];
#pragma unroll
      for (int k = 0; k < 16; ++k)
        x[k] = dequant_add_bias_h(unpack_i8(wi[k >> 2], k & 3), ds, bv[k]);
      float lo[8], hi[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        lo[k] = x[k];
        hi[k] = x[8 + k];
      }
      st8(dst, (long)s * d, lo);
      st8(dst, (long)s * d + 8, hi);
    }
  }
}

static int grid_for(long items) {
  long g = (items + 255) / 256;
  const long cap = 256L * 16;
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}
static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T>
int arrange_encself_qkv_i8I(int batch_token_num, int hidden_size, hipStream_t s,
                            const int8_t* ori_qkv, const T* qkv_bias, T* new_qkv,
                            long max_batch_dim, int batch_seq_len, int dim_per_head, int head_num,
                            float dequant_scale) {
  if (batch_token_num <= 0 || batch_seq_len <= 0 || head_num <= 0 || dim_per_head <= 0 ||
      hidden_size != dim_per_head * head_num || batch_token_num % batch_seq_len != 0 ||
      !ori_qkv || !qkv_bias || !new_qkv || max_batch_dim < (long)batch_token_num * hidden_size)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_encself_qkv_i8I: bad arguments");
  const long total = (long)batch_token_num * 3 * hidden_size;
  const bool vec = dim_per_head % 8 == 0 && max_batch_dim % 8 == 0 && al16(ori_qkv) &&
                   al16(qkv_bias) && al16(new_qkv);
  if constexpr (std::is_same<T, __half>::value) {
    const int batch = batch_token_num / batch_seq_len;
    if (vec && hidden_size % 128 == 0 && dim_per_head % 16 == 0 && 128 % dim_per_head == 0 &&
        batch_seq_len >= 32 && (long)batch * 3 * (hidden_size / 128) < (1L << 30)) {
      const int groups = hidden_size / 128;
      if (batch_seq_len > 64)
        arrange_qkv_heads_kernel<4><<<batch * 3 * groups, 256, 0, s>>>(
            ori_qkv, qkv_bias, new_qkv, max_batch_dim, batch_seq_len, dim_per_head, head_num,
            groups, dequant_scale);
      else
        arrange_qkv_heads_kernel<2><<<batch * 3 * groups, 256, 0, s>>>(
            ori_qkv, qkv_bias, new_qkv, max_batch_dim, batch_seq_len, dim_per_head, head_num,
            groups, dequant_scale);
      return lsh_check_launch("arrange_qkv_heads_kernel");
    }
  }
  if (vec)
    arrange_qkv_kernel<T, 8, false><<<grid_for(total / 8), 256, 0, s>>>(
        ori_qkv, qkv_bias, new_qkv, nullptr, nullptr, nullptr, nullptr, max_batch_dim, total / 8,
        batch_seq_len, dim_per_head, head_num, dequant_scale, 0.f);
  else
    arrange_qkv_kernel<T, 1, false><<<grid_for(total), 256, 0, s>>>(
        ori_qkv, qkv_bias, new_qkv, nullptr, nullptr, nullptr, nullptr, max_batch_dim, total,
        batch_seq_len, dim_per_head, head_num, dequant_scale, 0.f);
  return lsh_check_launch("arrange_qkv_kernel");
}

template <typename T>
int arrange_encself_qkv_i8I_i8O(int batch_token_num, int hidden_size, hipStream_t s,
                                const int8_t* ori_qkv, const T* qkv_bias, int8_t* new_q,
                                int8_t* new_k, int8_t* new_v, T* d_v, int batch_seq_len,
                                int dim_per_head, int head_num, float dequant_scale,
                                float quant_scale) {
  if (batch_token_num <= 0 || batch_seq_len <= 0 || head_num <= 0 || dim_per_head <= 0 ||
      hidden_size != dim_per_head * head_num || batch_token_num % batch_seq_len != 0 ||
      !ori_qkv || !qkv_bias || !new_q || !new_k || !new_v || !d_v)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_encself_qkv_i8I_i8O: bad arguments");
  const long total = (long)batch_token_num * 3 * hidden_size;
  const bool vec = dim_per_head % 8 == 0 && al16(ori_qkv) && al16(qkv_bias) && al16(new_q) &&
                   al16(new_k) && al16(new_v) && al16(d_v);
  if (vec)
    arrange_qkv_kernel<T, 8, true><<<grid_for(total / 8), 256, 0, s>>>(
        ori_qkv, qkv_bias, nullptr, new_q, new_k, new_v, d_v, 0, total / 8, batch_seq_len,
        dim_per_head, head_num, dequant_scale, quant_scale);
  else
    arrange_qkv_kernel<T, 1, true><<<grid_for(total), 256, 0, s>>>(
        ori_qkv, qkv_bias, nullptr, new_q, new_k, new_v, d_v, 0, total, batch_seq_len,
        dim_per_head, head_num, dequant_scale, quant_scale);
  return lsh_check_launch("arrange_qkv_kernel(i8O)");
}

// ---------------------------------------------------------------------------------
// [B, h, S, d] T  ->  [B*S, h*d] int8
template <typename T, int V>
__global__ void __launch_bounds__(256)
arrange_atten_output_kernel(const T* __restrict__ ori, int8_t* __restrict__ out, long total_v,
                            int beam_size, int d, int head_num, float qs) {
  const int hidden = d * head_num;
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; idx < total_v; idx += stride) {
    const long e = idx * V;  // flat output index
    const int i = (int)(e % hidden);
    const long tok = e / hidden;
    const int b = (int)(tok / beam_size), s = (int)(tok % beam_size);
    const int head = i / d, dim = i % d;
    const long src = (((long)b * head_num + head) * beam_size + s) * d + dim;
    if (V == 8) {
      float x[8];
      ld8(ori, src, x);
      *reinterpret_cast<uint2*>(out + e) = quant8(x, qs);
    } else {
      out[e] = (int8_t)float2int8(TT<T>::ld(ori, src), qs);
    }
  }
}

template <typename T>
int arrange_atten_output_i8O(int batch_token_num, int hidden_size, hipStream_t s, const T* ori_q,
                             int8_t* new_q, int beam_size, int dim_per_head, int head_num,
                             float quant_scale) {
  if (batch_token_num <= 0 || beam_size <= 0 || head_num <= 0 || dim_per_head <= 0 ||
      hidden_size != dim_per_head * head_num || batch_token_num % beam_size != 0 || !ori_q ||
      !new_q)
    return lsh_fail(LSH_ERR_INVALID, "ker_arrange_atten_output_i8O: bad arguments");
  const long total = (long)batch_token_num * hidden_size;
  if (dim_per_head % 8 == 0 && al16(ori_q) && al16(new_q))
    arrange_atten_output_kernel<T, 8><<<grid_for(total / 8), 256, 0, s>>>(
        ori_q, new_q, total / 8, beam_size, dim_per_head, head_num, quant_scale);
  else
    arrange_atten_output_kernel<T, 1><<<grid_for(total), 256, 0, s>>>(
        ori_q, new_q, total, beam_size, dim_per_head, head_num, quant_scale);
  return lsh_check_launch("arrange_atten_output_kernel");
}

// ---------------------------------------------------------------------------------
// token embedding from an int8 table + position embedding; writes the pad mask.
// vocab > 0: token ids are clamped into the table (an id outside it must not become a read
// outside the allocation); vocab <= 0: ids are used as they are, as the reference does.
template <typename T>
__global__ void __launch_bounds__(256)
enc_emb_kernel(const int8_t* __restrict__ token_emb, const T* __restrict__ pos_emb,
               const int* __restrict__ tokens, T* __restrict__ output, int* __restrict__ pad_mask,
               int pad_id, long total8, int seq_len, int hidden8, float scale, int vocab) {
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; idx < total8; idx += stride) {
    const int dim8 = (int)(idx % hidden8);
    const long tok_idx = idx / hidden8;
    const int seq = (int)(tok_idx % seq_len);
    int token = tokens[tok_idx];
    float v[8];
    if (token == pad_id) {
      if (dim8 == 0) pad_mask[tok_idx] = 1;
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = 0.f;
    } else {
      if (dim8 == 0) pad_mask[tok_idx] = 0;
      if (vocab > 0) token = min(max(token, 0), vocab - 1);
      float p[8];
      unpack8(*reinterpret_cast<const uint2*>(token_emb + ((long)token * hidden8 + dim8) * 8), v);
      ld8(pos_emb, ((long)seq * hidden8 + dim8) * 8, p);
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = v[k] * scale + p[k];
    }
    st8(output, idx * 8, v);
  }
}

template <typename T>
int enc_emb_i8I(const int8_t* token_emb, const T* pos_emb, const int* tokens, T* output,
                int* pad_mask, int pad_id, int batch_size, int seq_len, int hidden_dim,
                hipStream_t s, float dequant_scale, bool scaled, int vocab_size) {
  if (batch_size <= 0 || seq_len <= 0 || hidden_dim <= 0 || !token_emb || !pos_emb || !tokens ||
      !output || !pad_mask)
    return lsh_fail(LSH_ERR_INVALID, "launch_enc_emb_i8I: bad arguments");
  // the reference requires hidden % 8 (fp16) / % 4 (fp32); this kernel needs % 8 for both
  if (hidden_dim % 8 != 0) return lsh_fail(LSH_ERR_INVALID, "violate hidden_dim % 8 = 0");
  if (!al16(token_emb) || !al16(pos_emb) || !al16(output))
    return lsh_fail(LSH_ERR_INVALID, "launch_enc_emb_i8I: pointers must be 16-byte aligned");
  float scale = dequant_scale;
  if (scaled) scale *= sqrtf((float)hidden_dim);
  const long total8 = (long)batch_size * seq_len * (hidden_dim / 8);
  enc_emb_kernel<T><<<grid_for(total8), 256, 0, s>>>(token_emb, pos_emb, tokens, output, pad_mask,
                                                     pad_id, total8, seq_len, hidden_dim / 8,
                                                     scale, vocab_size);
  return lsh_check_launch("enc_emb_kernel");
}

#define LSH_INST(T)                                                                               \
  template int arrange_encself_qkv_i8I<T>(int, int, hipStream_t, const int8_t*, const T*, T*,     \
                                          long, int, int, int, float);                            \
  template int arrange_encself_qkv_i8I_i8O<T>(int, int, hipStream_t, const int8_t*, const T*,     \
                                              int8_t*, int8_t*, int8_t*, T*, int, int, int,       \
                                              float, float);                                      \
  template int arrange_atten_output_i8O<T>(int, int, hipStream_t, const T*, int8_t*, int, int,    \
                                           int, float);                                           \
  template int enc_emb_i8I<T>(const int8_t*, const T*, const int*, T*, int*, int, int, int, int,  \
                              hipStream_t, float, bool, int);
LSH_INST(float)
LSH_INST(__half)
#undef LSH_INST

}  // namespace lsh
