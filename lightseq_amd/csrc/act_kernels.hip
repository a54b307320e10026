// dequant + bias + GELU/ReLU + requant, int8 -> int8, one HBM pass (2 B/element).
//
// 16 consecutive codes per thread (one 16-byte load, one 16-byte store).
// Replaces inference/kernels/transformerKernels_int8.cc.cu:865-1078.
#include "ls_device.cuh"
#include "ls_launch.h"

namespace lsh {

template <typename T, int ACT>
__global__ void __launch_bounds__(256)
bias_act16_kernel(const int8_t* __restrict__ in, int8_t* __restrict__ out,
                  const T* __restrict__ bias, long n16, int feat, float ds, float qs,
                  float clip_max) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < n16; i += stride) {
    const long e = i * 16;
    const int col = (int)(e % feat);
    uint4 w = *reinterpret_cast<const uint4*>(in + e);
    uint32_t wi[4] = {w.x, w.y, w.z, w.w};
    uint32_t wo[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float b[4];
      ld4(bias, col + g * 4, b);
      int q[4];
#pragma unroll
      for (int k = 0; k < 4; ++k)
        q[k] = dequant_bias_act_requant<ACT>(unpack_i8(wi[g], k), ds, b[k], qs, clip_max);
      wo[g] = pack4_i8(q[0], q[1], q[2], q[3]);
    }
    *reinterpret_cast<uint4*>(out + e) = make_uint4(wo[0], wo[1], wo[2], wo[3]);
  }
}

template <typename T, int ACT>
__global__ void bias_act1_kernel(const int8_t* __restrict__ in, int8_t* __restrict__ out,
                                 const T* __restrict__ bias, long n, int feat, float ds, float qs,
                                 float clip_max) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    out[i] = (int8_t)dequant_bias_act_requant<ACT>((int)in[i], ds, TT<T>::ld(bias, i % feat), qs,
                                                   clip_max);
  }
}

template <typename T, int ACT>
static int launch_bias_act(int tokens, hipStream_t s, const int8_t* input, int8_t* output,
                           const T* bias, int feat, float ds, float qs, float clip_max) {
  if (tokens < 0 || feat <= 0 || (tokens > 0 && (!input || !output || !bias)))
    return lsh_fail(LSH_ERR_INVALID, "ker_bias_act_i8I_i8O: bad arguments");
  const long n = (long)tokens * feat;
  if (n == 0) return LSH_OK;
  const bool vec = feat % 16 == 0 && ((reinterpret_cast<uintptr_t>(input) |
                                       reinterpret_cast<uintptr_t>(output) |
                                       reinterpret_cast<uintptr_t>(bias)) & 15u) == 0;
  const long cap = 256L * 16;
  if (vec) {
    long n16 = n / 16;
    long g = (n16 + 255) / 256;
    bias_act16_kernel<T, ACT><<<(int)(g > cap ? cap : g), 256, 0, s>>>(input, output, bias, n16,
                                                                        feat, ds, qs, clip_max);
  } else {
    long g = (n + 255) / 256;
    bias_act1_kernel<T, ACT><<<(int)(g > cap ? cap : g), 256, 0, s>>>(input, output, bias, n, feat,
                                                                       ds, qs, clip_max);
  }
  return lsh_check_launch("bias_act_kernel");
}

template <typename T>
int bias_gelu_i8I_i8O(int tokens, hipStream_t s, const int8_t* input, int8_t* output,
                      const T* bias, int feature_dim, float dequant_scale, float quant_scale) {
  return launch_bias_act<T, kActGelu>(tokens, s, input, output, bias, feature_dim, dequant_scale,
                                   quant_scale, 0.f);
}

template <typename T>
int bias_relu_i8I_i8O(int tokens, hipStream_t s, const int8_t* input, int8_t* output,
                      const T* bias, int feature_dim, float dequant_scale, float quant_scale,
                      float clip_max, bool narrow_clip) {
  if (narrow_clip)
    return launch_bias_act<T, kActReluNarrow>(tokens, s, input, output, bias, feature_dim,
                                           dequant_scale, quant_scale, clip_max);
  return launch_bias_act<T, kActRelu>(tokens, s, input, output, bias, feature_dim, dequant_scale,
                                   quant_scale, clip_max);
}

#define LSH_INST(T)                                                                             \
  template int bias_gelu_i8I_i8O<T>(int, hipStream_t, const int8_t*, int8_t*, const T*, int,    \
                                    float, float);                                              \
  template int bias_relu_i8I_i8O<T>(int, hipStream_t, const int8_t*, int8_t*, const T*, int,    \
                                    float, float, float, bool);
LSH_INST(float)
LSH_INST(__half)
#undef LSH_INST

}  // namespace lsh
