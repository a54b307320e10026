// Device-side helpers shared by every gfx950 kernel of the int8 layer path.
// Wavefronts are 64 lanes wide; all reductions below are written for that.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lsh {

constexpr int kWave = 64;
constexpr float kLnEpsilon = 1e-12f;      // inference/kernels/transformerKernels.h:13
constexpr float kFloatInfNeg = -1.0e8f;   // inference/kernels/common.h:12

// ---- storage-type traits ---------------------------------------------------
template <typename T>
struct TT;
template <>
struct TT<float> {
  static constexpr bool is_half = false;
  __device__ static float ld(const float* p, long i) { return p[i]; }
  __device__ static void st(float* p, long i, float v) { p[i] = v; }
  // value as it would read back after a store
  __device__ static float rnd(float v) { return v; }
  // kernels/common.h:217-227 clamps half loads only
  __device__ static float safe(float v) { return v; }
};
template <>
struct TT<__half> {
  static constexpr bool is_half = true;
  __device__ static float ld(const __half* p, long i) { return __half2float(p[i]); }
  __device__ static void st(__half* p, long i, float v) { p[i] = __float2half_rn(v); }
  __device__ static float rnd(float v) { return __half2float(__float2half_rn(v)); }
  __device__ static float safe(float v) { return fmaxf(fminf(100000.f, v), -100000.f); }
};

// ---- scalar quantisers: inference/kernels/transformerKernels_int8.cc.cu:14-27
// (no FMA contraction in the three quantisers: the product is rounded before the
// +0.5, as written, so results do not depend on the compiler's fusing choices)
__device__ __forceinline__ int float2int8(float x, float quant_scale) {
#pragma clang fp contract(off)
  float i8_f = x * quant_scale;
  int i8 = (int)floorf(i8_f + 0.5f);
  return max(-127, min(127, i8));
}
__device__ __forceinline__ int posfloat2int8(float x, float quant_scale, float clip_max) {
#pragma clang fp contract(off)
  float i8_f = x * 2 * quant_scale - quant_scale * clip_max;
  int i8 = (int)floorf(i8_f + 0.5f);
  return max(-127, min(127, i8));
}
// int32 accumulator -> int8 code: the requantising GEMM epilogue.
__device__ __forceinline__ int requant_acc(int acc, float alpha) {
#pragma clang fp contract(off)
  float f = (float)acc * alpha;
  int q = (int)floorf(f + 0.5f);
  return max(-127, min(127, q));
}
// requant_acc in fewer instructions, bit for bit the same code: for every float y,
// floor(med3(y, -127, 127.5)) == clamp(floor(y), -127, 127), so the clamp can precede the one
// instruction that floors and converts.
__device__ __forceinline__ float requant_acc_clamped(int acc, float alpha) {
#pragma clang fp contract(off)
  float f = (float)acc * alpha;
  f = f + 0.5f;
  return __builtin_amdgcn_fmed3f(f, -127.f, 127.5f);
}
__device__ __forceinline__ int requant_acc_fast(int acc, float alpha) {
  int q;
  asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(q) : "v"(requant_acc_clamped(acc, alpha)));
  return q;
}
// four accumulators -> four codes in one word; the conversion writes its low byte in place
__device__ __forceinline__ uint32_t requant_acc_pack4(int a0, int a1, int a2, int a3, float alpha) {
  const float y0 = requant_acc_clamped(a0, alpha), y1 = requant_acc_clamped(a1, alpha);
  const float y2 = requant_acc_clamped(a2, alpha), y3 = requant_acc_clamped(a3, alpha);
  uint32_t p;
  asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD"
      : "=v"(p)
      : "v"(y0));
  asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD"
      : "+v"(p)
      : "v"(y1));
  asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD"
      : "+v"(p)
      : "v"(y2));
  asm("v_cvt_flr_i32_f32_sdwa %0, %1 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD"
      : "+v"(p)
      : "v"(y3));
  return p;
}
// inference/kernels/common.h:17-23
__device__ __forceinline__ float gelu_tanh(float x) {
  float cdf = 0.5f * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
  return x * cdf;
}

// tanh-form GELU written as x * sigmoid(2u): 0.5 * (1 + tanh(u)) == 1 / (1 + exp(-2u));
// one hardware exp and one reciprocal instead of a tanhf call.
__device__ __forceinline__ float gelu_sigmoid_form(float x) {
  float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return x * __frcp_rn(1.0f + __expf(-2.0f * u));
}

enum ActKind { kActGelu = 0, kActRelu = 1, kActReluNarrow = 2 };

// int8 code -> dequant + bias -> activation -> int8 code
// (inference/kernels/transformerKernels_int8.cc.cu:865-1078).  Shared by the stand-alone
// kernel and the fused GEMM epilogue so both produce the same bits.
template <int ACT>
__device__ __forceinline__ int dequant_bias_act_requant(int q, float dequant_scale, float bias,
                                                        float quant_scale, float clip_max) {
  float x;
  {
#pragma clang fp contract(off)
    x = (float)q * dequant_scale + bias;
  }
  if (ACT == kActGelu) return float2int8(gelu_sigmoid_form(x), quant_scale);
  float r = fmaxf(x, 0.f);
  if (ACT == kActReluNarrow) return posfloat2int8(r, quant_scale, clip_max);
  return float2int8(r, quant_scale);
}

// fp16 head-split value: T(q * dequant_scale) + bias as a half add
// (inference/kernels/transformerKernels_int8.cc.cu:1140-1145); the caller rounds the
// returned float to fp16.
__device__ __forceinline__ float dequant_add_bias_h(int q, float dequant_scale, float bias) {
  return __half2float(__float2half_rn((float)q * dequant_scale)) + bias;
}

__device__ __forceinline__ uint32_t pack4_i8(int a, int b, int c, int d) {
  return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
         ((uint32_t)(d & 0xff) << 24);
}
__device__ __forceinline__ int unpack_i8(uint32_t w, int i) {
  return (int)(int8_t)((w >> (8 * i)) & 0xff);
}

// ---- vector views ------------------------------------------------------------
struct __align__(8) half4_t {
  __half v[4];
};
struct __align__(16) half8_t {
  __half v[8];
};

// load/store 4 consecutive T as floats
__device__ __forceinline__ void ld4(const float* p, long i, float (&o)[4]) {
  float4 t = *reinterpret_cast<const float4*>(p + i);
  o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
}
__device__ __forceinline__ void ld4(const __half* p, long i, float (&o)[4]) {
  half4_t t = *reinterpret_cast<const half4_t*>(p + i);
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = __half2float(t.v[k]);
}
// Four consecutive T as raw words, to be converted after pin4(): between the two the caller
// requests whatever else it loads.  pin4() makes the words opaque to the compiler, which
// otherwise sinks a load whose values are used under a condition into that branch, where it
// is followed by its wait -- one memory round trip after the other.
struct Raw4F { float4 v; };
struct Raw4H { uint2 v; };
__device__ __forceinline__ Raw4F ld4_raw(const float* p, long i) {
  return Raw4F{*reinterpret_cast<const float4*>(p + i)};
}
__device__ __forceinline__ Raw4H ld4_raw(const __half* p, long i) {
  return Raw4H{*reinterpret_cast<const uint2*>(p + i)};
}
__device__ __forceinline__ void pin4(Raw4F& a, Raw4F& b, Raw4F& c, Raw4F& d) {
  asm volatile("" : "+v"(a.v.x), "+v"(a.v.y), "+v"(a.v.z), "+v"(a.v.w), "+v"(b.v.x), "+v"(b.v.y),
               "+v"(b.v.z), "+v"(b.v.w), "+v"(c.v.x), "+v"(c.v.y), "+v"(c.v.z), "+v"(c.v.w),
               "+v"(d.v.x), "+v"(d.v.y), "+v"(d.v.z), "+v"(d.v.w));
}
__device__ __forceinline__ void pin4(Raw4H& a, Raw4H& b, Raw4H& c, Raw4H& d) {
  asm volatile("" : "+v"(a.v.x), "+v"(a.v.y), "+v"(b.v.x), "+v"(b.v.y), "+v"(c.v.x), "+v"(c.v.y),
               "+v"(d.v.x), "+v"(d.v.y));
}
__device__ __forceinline__ void cvt4(const Raw4F& r, float (&o)[4]) {
  o[0] = r.v.x; o[1] = r.v.y; o[2] = r.v.z; o[3] = r.v.w;
}
__device__ __forceinline__ void cvt4(const Raw4H& r, float (&o)[4]) {
  half4_t t;
  __builtin_memcpy(&t, &r.v, sizeof(t));
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = __half2float(t.v[k]);
}
__device__ __forceinline__ void st4(float* p, long i, const float (&o)[4]) {
  *reinterpret_cast<float4*>(p + i) = make_float4(o[0], o[1], o[2], o[3]);
}
__device__ __forceinline__ void st4(__half* p, long i, const float (&o)[4]) {
  half4_t t;
#pragma unroll
  for (int k = 0; k < 4; ++k) t.v[k] = __float2half_rn(o[k]);
  *reinterpret_cast<half4_t*>(p + i) = t;
}

// ---- wavefront reductions ------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = kWave / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, kWave));
  return v;
}

// The same over DPP permutations and lane reads: no LDS permute instructions and a much
// shorter dependent chain (quad, 8 lanes, 16 lanes, then the four rows of the wavefront
// pairwise).  Another order of additions than wave_sum; every lane gets the result.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane l of a row of 16 reads lane 7 - l of its half
constexpr int kDppMirror = 0x140;      // ... lane 15 - l of its row
__device__ __forceinline__ float lane_read(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v += dpp_f<kDppXor1>(v);
  v += dpp_f<kDppXor2>(v);
  v += dpp_f<kDppHalfMirror>(v);
  v += dpp_f<kDppMirror>(v);
  return (lane_read(v, 0) + lane_read(v, 16)) + (lane_read(v, 32) + lane_read(v, 48));
}
__device__ __forceinline__ float wave_max_dpp(float v) {
  v = fmaxf(v, dpp_f<kDppXor1>(v));
  v = fmaxf(v, dpp_f<kDppXor2>(v));
  v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_f<kDppMirror>(v));
  return fmaxf(fmaxf(lane_read(v, 0), lane_read(v, 16)), fmaxf(lane_read(v, 32), lane_read(v, 48)));
}
// Block-wide forms with one barrier: `red` (16 floats of LDS) must not be in use by an
// earlier reduction that other wavefronts may still be reading (give each call its own).
__device__ __forceinline__ float block_sum_dpp(float v, float* red) {
  v = wave_sum_dpp(v);
  const int nw = (blockDim.x + kWave - 1) >> 6;
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
  for (int i = 1; i < nw; ++i) r += red[i];
  return r;
}
__device__ __forceinline__ float block_max_dpp(float v, float* red) {
  v = wave_max_dpp(v);
  const int nw = (blockDim.x + kWave - 1) >> 6;
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
  for (int i = 1; i < nw; ++i) r = fmaxf(r, red[i]);
  return r;
}

// Block-wide reductions for blocks of up to 1024 threads (16 wavefronts).
// `red` must point to at least 16 floats of LDS.  All threads get the result.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x >> 6;
  const int nw = (blockDim.x + kWave - 1) >> 6;
  __syncthreads();  // protect `red` from a previous use
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += red[i];
  return r;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x >> 6;
  const int nw = (blockDim.x + kWave - 1) >> 6;
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float r = red[0];
  for (int i = 1; i < nw; ++i) r = fmaxf(r, red[i]);
  return r;
}

}  // namespace lsh
