// LayerNorm family of the int8 layer path: dequant + residual (+colsum) +
// LayerNorm + quant, one HBM pass.
//
// Layout: one 64-lane wavefront owns one token row and keeps it in registers
// (4 consecutive elements per lane per step, so a row of `hidden` elements takes
// ceil(hidden/256) steps); mean and variance are the reference's two-pass form,
// reduced with cross-lane shuffles.  Four rows per 256-thread workgroup.
//
// Replaces inference/kernels/transformerKernels_int8.cc.cu:149-863.
#include "ls_device.cuh"
#include "ls_launch.h"

namespace lsh {

enum LnMode {
  kLnFirst = 0,    // ker_norm_layer_resual_i8O      (:149-316)
  kLnResQuant = 1, // ker_residual_bias_ln_i{8,32}I_i8O (:318-705)
  kLnResOut = 2    // ker_residual_bias_ln_i32I      (:707-863)
};

__device__ __forceinline__ void ld4_acc(const int8_t* p, long i, float (&o)[4]) {
  uint32_t w = *reinterpret_cast<const uint32_t*>(p + i);
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = (float)unpack_i8(w, k);
}
__device__ __forceinline__ void ld4_acc(const int32_t* p, long i, float (&o)[4]) {
  int4 w = *reinterpret_cast<const int4*>(p + i);
  o[0] = (float)w.x; o[1] = (float)w.y; o[2] = (float)w.z; o[3] = (float)w.w;
}

// Vectorised kernel.  Preconditions (checked by the launcher): hidden % 4 == 0,
// hidden <= ITER * 256, all pointers 16-byte aligned.
template <typename T, typename AccT, int MODE, int ITER>
__global__ void __launch_bounds__(256)
ln_rows_kernel(const AccT* __restrict__ gemm_out, T* residual, T* out_t,
               int8_t* __restrict__ out_q, const T* __restrict__ scale,
               const T* __restrict__ bias, const T* __restrict__ residual_bias,
               const T* __restrict__ colsum, int tokens, int hidden, float dequant_scale,
               float quant_scale, int is_post_ln) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= tokens) return;
  const long base = (long)row * hidden;

  float x[ITER][4];
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int e = (it * 64 + lane) * 4;
    if (e < hidden) {
      float r[4];
      ld4(residual, base + e, r);
      if (MODE == kLnFirst) {
#pragma unroll
        for (int k = 0; k < 4; ++k) x[it][k] = TT<T>::safe(r[k]);
      } else {
        float a[4];
        ld4_acc(gemm_out, base + e, a);
#pragma unroll
        for (int k = 0; k < 4; ++k) x[it][k] = a[k] * dequant_scale + TT<T>::safe(r[k]);
        if (colsum != nullptr) {
          float c[4];
          ld4(colsum, e, c);
#pragma unroll
          for (int k = 0; k < 4; ++k) x[it][k] += TT<T>::safe(c[k]);
        }
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) sum += x[it][k];
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) x[it][k] = 0.f;
    }
  }
  const float mean = wave_sum(sum) / (float)hidden;
  float var = 0.f;
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int e = (it * 64 + lane) * 4;
    if (e < hidden) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float t = x[it][k] - mean;
        var += t * t;
      }
    }
  }
  const float rstd = rsqrtf(wave_sum(var) / (float)hidden + kLnEpsilon);

#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int e = (it * 64 + lane) * 4;
    if (e < hidden) {
      float g[4], b[4], o[4];
      ld4(scale, e, g);
      ld4(bias, e, b);
#pragma unroll
      for (int k = 0; k < 4; ++k)
        o[k] = (x[it][k] - mean) * rstd * TT<T>::safe(g[k]) + TT<T>::safe(b[k]);
      if (MODE == kLnResOut) {
        st4(out_t, base + e, o);
      } else {
        *reinterpret_cast<uint32_t*>(out_q + base + e) =
            pack4_i8(float2int8(o[0], quant_scale), float2int8(o[1], quant_scale),
                     float2int8(o[2], quant_scale), float2int8(o[3], quant_scale));
        float rb[4] = {0.f, 0.f, 0.f, 0.f};
        if (residual_bias != nullptr) ld4(residual_bias, e, rb);
        float w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float keep = is_post_ln ? o[k] : x[it][k];
          // first-layer kernel adds in float and rounds once; the residual
          // kernels round to T first and add in T (a half add for fp16).
          w[k] = (MODE == kLnFirst) ? keep + rb[k] : TT<T>::rnd(keep) + rb[k];
        }
        st4(residual, base + e, w);
      }
    }
  }
}

// Any hidden size / alignment: one workgroup per row, row staged in LDS.
template <typename T, typename AccT, int MODE>
__global__ void ln_rows_generic_kernel(const AccT* __restrict__ gemm_out, T* residual, T* out_t,
                                       int8_t* __restrict__ out_q, const T* __restrict__ scale,
                                       const T* __restrict__ bias,
                                       const T* __restrict__ residual_bias,
                                       const T* __restrict__ colsum, int hidden,
                                       float dequant_scale, float quant_scale, int is_post_ln) {
  extern __shared__ float s_row[];
  __shared__ float red[16];
  const long base = (long)blockIdx.x * hidden;
  float sum = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = TT<T>::safe(TT<T>::ld(residual, base + i));
    if (MODE != kLnFirst) {
      v = (float)gemm_out[base + i] * dequant_scale + v;
      if (colsum != nullptr) v += TT<T>::safe(TT<T>::ld(colsum, i));
    }
    s_row[i] = v;
    sum += v;
  }
  const float mean = block_sum(sum, red) / (float)hidden;
  float var = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float t = s_row[i] - mean;
    var += t * t;
  }
  const float rstd = rsqrtf(block_sum(var, red) / (float)hidden + kLnEpsilon);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float o = (s_row[i] - mean) * rstd * TT<T>::safe(TT<T>::ld(scale, i)) +
              TT<T>::safe(TT<T>::ld(bias, i));
    if (MODE == kLnResOut) {
      TT<T>::st(out_t, base + i, o);
    } else {
      out_q[base + i] = (int8_t)float2int8(o, quant_scale);
      float rb = residual_bias != nullptr ? TT<T>::ld(residual_bias, i) : 0.f;
      float keep = is_post_ln ? o : s_row[i];
      TT<T>::st(residual, base + i, (MODE == kLnFirst) ? keep + rb : TT<T>::rnd(keep) + rb);
    }
  }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T, typename AccT, int MODE>
static int launch_ln(const AccT* gemm_out, T* residual, T* out_t, int8_t* out_q, const T* scale,
                     const T* bias, const T* residual_bias, const T* colsum, int tokens,
                     int hidden, float dequant_scale, float quant_scale, int is_post_ln,
                     hipStream_t stream) {
  if (tokens <= 0 || hidden <= 0) return lsh_fail(LSH_ERR_INVALID, "layer norm: empty shape");
  const bool vec_ok = hidden % 4 == 0 && hidden <= 2048 && aligned16(gemm_out) &&
                      aligned16(residual) && aligned16(out_t) && aligned16(out_q) &&
                      aligned16(scale) && aligned16(bias) && aligned16(residual_bias) &&
                      aligned16(colsum);
  if (!vec_ok) {
    if ((size_t)hidden * sizeof(float) > 160 * 1024 - 256)
      return lsh_fail(LSH_ERR_UNSUPPORTED, "layer norm: hidden size too large");
    ln_rows_generic_kernel<T, AccT, MODE>
        <<<tokens, 256, (size_t)hidden * sizeof(float), stream>>>(
            gemm_out, residual, out_t, out_q, scale, bias, residual_bias, colsum, hidden,
            dequant_scale, quant_scale, is_post_ln);
    return lsh_check_launch("ln_rows_generic_kernel");
  }
  const int grid = (tokens + 3) / 4;
#define LSH_LN_CASE(IT)                                                                        \
  ln_rows_kernel<T, AccT, MODE, IT><<<grid, 256, 0, stream>>>(                                 \
      gemm_out, residual, out_t, out_q, scale, bias, residual_bias, colsum, tokens, hidden,    \
      dequant_scale, quant_scale, is_post_ln)
  const int iters = (hidden + 255) / 256;
  switch (iters) {
    case 1: LSH_LN_CASE(1); break;
    case 2: LSH_LN_CASE(2); break;
    case 3: LSH_LN_CASE(3); break;
    case 4: LSH_LN_CASE(4); break;
    case 5: case 6: LSH_LN_CASE(6); break;
    default: LSH_LN_CASE(8); break;
  }
#undef LSH_LN_CASE
  return lsh_check_launch("ln_rows_kernel");
}

template <typename T>
int norm_layer_resual_i8O(int token_num, int hidden_size, hipStream_t stream, T* input,
                          int8_t* output, const T* scale, const T* bias, const T* residual_bias,
                          float quant_scale, bool is_post_ln) {
  if (!input || !output || !scale || !bias || !residual_bias)
    return lsh_fail(LSH_ERR_INVALID, "ker_norm_layer_resual_i8O: null pointer");
  return launch_ln<T, int8_t, kLnFirst>(nullptr, input, nullptr, output, scale, bias,
                                        residual_bias, nullptr, token_num, hidden_size, 0.f,
                                        quant_scale, is_post_ln, stream);
}

template <typename T, typename AccT>
int residual_bias_ln_i8O(const AccT* input, const T* scale, const T* bias, const T* residual_bias,
                         int8_t* output, T* residual, int batch_tokens, int hidden_size,
                         float dequant_scale, float quant_scale, hipStream_t stream,
                         bool is_post_ln, const T* colsum) {
  if (!input || !output || !scale || !bias || !residual)
    return lsh_fail(LSH_ERR_INVALID, "ker_residual_bias_ln_*_i8O: null pointer");
  return launch_ln<T, AccT, kLnResQuant>(input, residual, nullptr, output, scale, bias,
                                         residual_bias, colsum, batch_tokens, hidden_size,
                                         dequant_scale, quant_scale, is_post_ln, stream);
}

template <typename T>
int residual_bias_ln_i32I(const int32_t* input, const T* scale, const T* bias, const T* residual,
                          T* output, int batch_tokens, int hidden_size, float dequant_scale,
                          hipStream_t stream, const T* colsum) {
  if (!input || !output || !scale || !bias || !residual)
    return lsh_fail(LSH_ERR_INVALID, "ker_residual_bias_ln_i32I: null pointer");
  // the kernel only reads `residual`; output may alias it (the reference calls it in place)
  return launch_ln<T, int32_t, kLnResOut>(input, const_cast<T*>(residual), output, nullptr, scale,
                                          bias, nullptr, colsum, batch_tokens, hidden_size,
                                          dequant_scale, 0.f, 0, stream);
}

#define LSH_INST(T)                                                                              \
  template int norm_layer_resual_i8O<T>(int, int, hipStream_t, T*, int8_t*, const T*, const T*,  \
                                        const T*, float, bool);                                  \
  template int residual_bias_ln_i8O<T, int8_t>(const int8_t*, const T*, const T*, const T*,      \
                                               int8_t*, T*, int, int, float, float, hipStream_t, \
                                               bool, const T*);                                  \
  template int residual_bias_ln_i8O<T, int32_t>(const int32_t*, const T*, const T*, const T*,    \
                                                int8_t*, T*, int, int, float, float,             \
                                                hipStream_t, bool, const T*);                    \
  template int residual_bias_ln_i32I<T>(const int32_t*, const T*, const T*, const T*, T*, int,   \
                                        int, float, hipStream_t, const T*);
LSH_INST(float)
LSH_INST(__half)
#undef LSH_INST

}  // namespace lsh
