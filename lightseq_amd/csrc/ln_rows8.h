// The row routine of the 8-wide layer-norm kernels (dequantise + residual (+ column sums) +
// LayerNorm + quantise of one token row held by LPR lanes), shared by the stand-alone kernel,
// the out-projection kernel that ends in it (ln_kernels.hip) and the per-XCD feed-forward
// segment (xcd_ffn_kernels.hip).  Replaces inference/kernels/transformerKernels_int8.cc.cu:
// 149-863.
#pragma once
#include "ls_device.h"

namespace lsh {

enum LnMode {
  kLnFirst = 0,    // ker_norm_layer_resual_i8O      (:149-316)
  kLnResQuant = 1, // ker_residual_bias_ln_i{8,32}I_i8O (:318-705)
  kLnResOut = 2    // ker_residual_bias_ln_i32I      (:707-863)
};

// 8 consecutive elements per lane per step (one 16-byte load of fp16 data, 8 bytes of int8
// codes, two 16-byte loads of int32 accumulators); LPR lanes share a row, so a wavefront
// covers 64/LPR rows and a workgroup 4 * 64/LPR.  All loads of a lane are issued before the
// first reduction.  `nparts` int32 accumulator planes `part_stride` elements apart are
// summed first (the split-K form of the int32 GEMM); the sum of integers is exact.
// Preconditions (checked by the launcher): hidden % 8 == 0, hidden <= LPR * 8 * ITER,
// 16-byte aligned pointers.
__device__ __forceinline__ void ld8_acc(const int8_t* p, long i, float (&o)[8]) {
  uint2 w = *reinterpret_cast<const uint2*>(p + i);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    o[k] = (float)unpack_i8(w.x, k);
    o[4 + k] = (float)unpack_i8(w.y, k);
  }
}
__device__ __forceinline__ void ld8_acc(const int32_t* p, long i, int (&o)[8]) {
  int4 a = *reinterpret_cast<const int4*>(p + i);
  int4 b = *reinterpret_cast<const int4*>(p + i + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
  o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
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
// Eight consecutive elements as raw words (converted after every load of the row has been
// requested) and the statement that makes the words opaque to the compiler, which otherwise
// sinks a load into the branch that uses its values, where it is followed by its wait.
struct Raw8F { float4 a, b; };
struct Raw8H { uint4 a; };
struct Raw8I { int4 a, b; };
struct Raw8C { uint2 a; };
__device__ __forceinline__ Raw8F ld8_raw(const float* p, long i) {
  return Raw8F{*reinterpret_cast<const float4*>(p + i), *reinterpret_cast<const float4*>(p + i + 4)};
}
__device__ __forceinline__ Raw8H ld8_raw(const __half* p, long i) {
  return Raw8H{*reinterpret_cast<const uint4*>(p + i)};
}
__device__ __forceinline__ Raw8I ld8_raw(const int32_t* p, long i) {
  return Raw8I{*reinterpret_cast<const int4*>(p + i), *reinterpret_cast<const int4*>(p + i + 4)};
}
__device__ __forceinline__ Raw8C ld8_raw(const int8_t* p, long i) {
  return Raw8C{*reinterpret_cast<const uint2*>(p + i)};
}
__device__ __forceinline__ void pin8(Raw8F& r) {
  asm volatile("" : "+v"(r.a.x), "+v"(r.a.y), "+v"(r.a.z), "+v"(r.a.w), "+v"(r.b.x), "+v"(r.b.y),
               "+v"(r.b.z), "+v"(r.b.w));
}
__device__ __forceinline__ void pin8(Raw8H& r) {
  asm volatile("" : "+v"(r.a.x), "+v"(r.a.y), "+v"(r.a.z), "+v"(r.a.w));
}
__device__ __forceinline__ void pin8(Raw8I& r) {
  asm volatile("" : "+v"(r.a.x), "+v"(r.a.y), "+v"(r.a.z), "+v"(r.a.w), "+v"(r.b.x), "+v"(r.b.y),
               "+v"(r.b.z), "+v"(r.b.w));
}
__device__ __forceinline__ void pin8(Raw8C& r) { asm volatile("" : "+v"(r.a.x), "+v"(r.a.y)); }
__device__ __forceinline__ void cvt8(const Raw8F& r, float (&o)[8]) {
  o[0] = r.a.x; o[1] = r.a.y; o[2] = r.a.z; o[3] = r.a.w;
  o[4] = r.b.x; o[5] = r.b.y; o[6] = r.b.z; o[7] = r.b.w;
}
__device__ __forceinline__ void cvt8(const Raw8H& r, float (&o)[8]) {
  half8_t t;
  __builtin_memcpy(&t, &r.a, sizeof(t));
#pragma unroll
  for (int k = 0; k < 8; ++k) o[k] = __half2float(t.v[k]);
}
__device__ __forceinline__ void cvt8(const Raw8I& r, int (&o)[8]) {
  o[0] = r.a.x; o[1] = r.a.y; o[2] = r.a.z; o[3] = r.a.w;
  o[4] = r.b.x; o[5] = r.b.y; o[6] = r.b.z; o[7] = r.b.w;
}
__device__ __forceinline__ void cvt8(const Raw8C& r, float (&o)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    o[k] = (float)unpack_i8(r.a.x, k);
    o[4 + k] = (float)unpack_i8(r.a.y, k);
  }
}
template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
  for (int m = LPR / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}

// One row of the 8-wide kernel: `sub` is the lane's index among the LPR lanes of the row,
// `live` false for a row beyond the tensor (its lanes still take part in the shuffles).
// gemm_out is read at gemm_out[row * hidden + column] and may point anywhere a flat load
// reaches (the fused GEMM + LayerNorm kernel passes a tile staged in LDS).
template <typename T, typename AccT, int MODE, int LPR, int ITER>
__device__ __forceinline__ void
ln_rows8_row(int row, bool live, int sub, const AccT* __restrict__ gemm_out, T* residual, T* out_t,
             int8_t* __restrict__ out_q, const T* __restrict__ scale, const T* __restrict__ bias,
             const T* __restrict__ residual_bias, const T* __restrict__ colsum, int hidden,
             float dequant_scale, float quant_scale, int is_post_ln, int nparts, long part_stride,
             const half8_t* pre_res = nullptr, int dead_row = 0) {
  // pre_res (fp16 only): the lane's ITER residual chunks, already loaded by the caller.
  // dead_row: the row whose addresses a lane without a row reads (and drops); a caller that
  // hands over a staged tile names a row of the tile.
  const long base = (long)(live ? row : dead_row) * hidden;

  float x[ITER][8];
  // Every load of the row -- parameters, residual, accumulator, column sums -- is requested
  // before the first value is used: no branch around a load (columns beyond the row and rows
  // beyond the tensor are clamped, optional operands read through a pointer that is always
  // valid, and what they bring is dropped), a scheduling barrier after the last request, and
  // only then the statements that make the values visible to the arithmetic.  Written with
  // conditions around the loads, the compiler put each load next to its use: six to nine
  // memory round trips in a row instead of one.
  const bool has_rb = MODE != kLnResOut && residual_bias != nullptr;
  const bool has_cs = MODE != kLnFirst && colsum != nullptr;
  const bool own_res = !(sizeof(T) == 2 && pre_res != nullptr);
  const T* rbp = has_rb ? residual_bias : scale;
  const T* csp = has_cs ? colsum : scale;
  decltype(ld8_raw(scale, 0)) g_raw[ITER], b_raw[ITER], rb_raw[ITER], cs_raw[ITER], r_raw[ITER];
  decltype(ld8_raw(gemm_out, 0)) a_raw[ITER];
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int e = min((it * LPR + sub) * 8, hidden - 8);
    g_raw[it] = ld8_raw(scale, e);
    b_raw[it] = ld8_raw(bias, e);
    rb_raw[it] = ld8_raw(rbp, e);
    cs_raw[it] = ld8_raw(csp, e);
    r_raw[it] = ld8_raw(own_res ? residual + base + e : scale, 0);
    if (MODE != kLnFirst) a_raw[it] = ld8_raw(gemm_out, base + e);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    pin8(g_raw[it]);
    pin8(b_raw[it]);
    pin8(rb_raw[it]);
    pin8(cs_raw[it]);
    pin8(r_raw[it]);
    if (MODE != kLnFirst) pin8(a_raw[it]);
  }
  float gs[ITER][8], bs[ITER][8], rbs[ITER][8];
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int e = (it * LPR + sub) * 8;
    cvt8(g_raw[it], gs[it]);
    cvt8(b_raw[it], bs[it]);
    cvt8(rb_raw[it], rbs[it]);
#pragma unroll
    for (int k = 0; k < 8; ++k) rbs[it][k] = has_rb ? rbs[it][k] : 0.f;
    if (e < hidden && live) {
      float r[8];
      if (own_res) {
        cvt8(r_raw[it], r);
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) r[k] = __half2float(pre_res[it].v[k]);
      }
      if (MODE == kLnFirst) {
#pragma unroll
        for (int k = 0; k < 8; ++k) x[it][k] = TT<T>::safe(r[k]);
      } else {
        float a[8];
        if constexpr (sizeof(AccT) == 4) {
          // further planes in a rolled loop: launches of a few rows, where the planes come
          // from, use the row kernel, and this one stays small
          int acc[8];
          cvt8(a_raw[it], acc);
          for (int p = 1; p < nparts; ++p) {
            int more[8];
            ld8_acc(gemm_out + p * part_stride, base + e, more);
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[k] += more[k];
          }
#pragma unroll
          for (int k = 0; k < 8; ++k) a[k] = (float)acc[k];
        } else {
          cvt8(a_raw[it], a);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) x[it][k] = a[k] * dequant_scale + TT<T>::safe(r[k]);
        if (has_cs) {
          float c[8];
          cvt8(cs_raw[it], c);
#pragma unroll
          for (int k = 0; k < 8; ++k) x[it][k] += TT<T>::safe(c[k]);
        }
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) sum += x[it][k];
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) x[it][k] = 0.f;
    }
  }
  const float mean = row_sum<LPR>(sum) / (float)hidden;
  float var = 0.f;
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int e = (it * LPR + sub) * 8;
    if (e < hidden) {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        float t = x[it][k] - mean;
        var += t * t;
      }
    }
  }
  const float rstd = rsqrtf(row_sum<LPR>(var) / (float)hidden + kLnEpsilon);
  if (!live) return;

#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    const int e = (it * LPR + sub) * 8;
    if (e < hidden) {
      float o[8];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        o[k] = (x[it][k] - mean) * rstd * TT<T>::safe(gs[it][k]) + TT<T>::safe(bs[it][k]);
      if (MODE == kLnResOut) {
        st8(out_t, base + e, o);
      } else {
        uint2 packed;
        packed.x = pack4_i8(float2int8(o[0], quant_scale), float2int8(o[1], quant_scale),
                            float2int8(o[2], quant_scale), float2int8(o[3], quant_scale));
        packed.y = pack4_i8(float2int8(o[4], quant_scale), float2int8(o[5], quant_scale),
                            float2int8(o[6], quant_scale), float2int8(o[7], quant_scale));
        *reinterpret_cast<uint2*>(out_q + base + e) = packed;
        float w[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          float keep = is_post_ln ? o[k] : x[it][k];
          w[k] = (MODE == kLnFirst) ? keep + rbs[it][k] : TT<T>::rnd(keep) + rbs[it][k];
        }
        st8(residual, base + e, w);
      }
    }
  }
}

}  // namespace lsh
