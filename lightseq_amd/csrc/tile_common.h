// Device helpers shared by the int8 GEMM tile kernels, the fused attention kernels and the
// kernel that does both: MFMA vector types, the XOR swizzle of 128-byte LDS rows, the
// requantising pack, int8 -> fp16 dequantisation, and the attention of one block of up to
// 128 keys held in LDS.
#pragma once
#include "ls_device.h"

namespace lsh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 128;  // bytes of K per LDS stage

// swizzle keys (3 bits) of a tile row, for the activation tile (rows read in natural
// order) and the weight tile (rows read in sigma order)
__device__ __forceinline__ int key_act(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int key_wgt(int row) { return ((row >> 1) & 3) | (((row >> 4) & 1) << 2); }
// MFMA row r (0..31) of the weight operand -> local column of C, chosen so that the
// accumulators c[0..15] of lane (l%32, g=l/32) are columns 16g .. 16g+15.
__device__ __forceinline__ int sigma(int r) { return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3); }

__device__ __forceinline__ uint4 requant16_packed(const v16i& c, float alpha) {
  uint4 o;
  o.x = requant_acc_pack4(c[0], c[1], c[2], c[3], alpha);
  o.y = requant_acc_pack4(c[4], c[5], c[6], c[7], alpha);
  o.z = requant_acc_pack4(c[8], c[9], c[10], c[11], alpha);
  o.w = requant_acc_pack4(c[12], c[13], c[14], c[15], alpha);
  return o;
}


template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}


typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float round_h(float x) { return (float)(_Float16)x; }


template <int N>
__device__ __forceinline__ float ubyte_f32(uint32_t w) {  // one v_cvt_f32_ubyteN
  return (float)((w >> (8 * N)) & 0xffu);
}

// 16 int8 codes -> 16 fp16 values half(half(code * dq) + bias)
__device__ __forceinline__ void dequant16_bias(const uint4& w, const _Float16* __restrict__ bias,
                                               float dq, v8h& lo, v8h& hi) {
  // float(code) * dq == fma(float(code + 128), dq, -128 * dq): the product is exact before
  // its single rounding either way, and -128 * dq is exact.  half(x) + half(b) in fp16
  // arithmetic == half(float(x) + float(b)): the float sum of two halfs is exact unless
  // one is below a quarter of the other's last place, where both round to the larger one.
  const v8h b0 = *reinterpret_cast<const v8h*>(bias);
  const v8h b1 = *reinterpret_cast<const v8h*>(bias + 8);
  const float off = -128.f * dq;
  const uint32_t u[4] = {w.x ^ 0x80808080u, w.y ^ 0x80808080u, w.z ^ 0x80808080u,
                         w.w ^ 0x80808080u};
  v8h xl, xh;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    xl[4 * j + 0] = (_Float16)fmaf(ubyte_f32<0>(u[j]), dq, off);
    xl[4 * j + 1] = (_Float16)fmaf(ubyte_f32<1>(u[j]), dq, off);
    xl[4 * j + 2] = (_Float16)fmaf(ubyte_f32<2>(u[j]), dq, off);
    xl[4 * j + 3] = (_Float16)fmaf(ubyte_f32<3>(u[j]), dq, off);
    xh[4 * j + 0] = (_Float16)fmaf(ubyte_f32<0>(u[2 + j]), dq, off);
    xh[4 * j + 1] = (_Float16)fmaf(ubyte_f32<1>(u[2 + j]), dq, off);
    xh[4 * j + 2] = (_Float16)fmaf(ubyte_f32<2>(u[2 + j]), dq, off);
    xh[4 * j + 3] = (_Float16)fmaf(ubyte_f32<3>(u[2 + j]), dq, off);
  }
  lo = xl + b0;
  hi = xh + b1;
}

// 16 int32 accumulators -> the 16 fp16 values half(half(code * dq) + bias) of their int8 codes
// code = requant_acc(acc, alpha), without forming the codes as bytes: floor(med3(y, -127, 127.5))
// is the code as a float, and half(float(code) * dq) is what dequant16_bias computes from it.
__device__ __forceinline__ void requant_dequant16_bias(const v16i& c, float alpha,
                                                       const _Float16* __restrict__ bias, float dq,
                                                       v8h& lo, v8h& hi) {
  const v8h b0 = *reinterpret_cast<const v8h*>(bias);
  const v8h b1 = *reinterpret_cast<const v8h*>(bias + 8);
  v8h xl, xh;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    xl[j] = (_Float16)(floorf(requant_acc_clamped(c[j], alpha)) * dq);
    xh[j] = (_Float16)(floorf(requant_acc_clamped(c[8 + j], alpha)) * dq);
  }
  lo = xl + b0;
  hi = xh + b1;
}

// 8 int8 codes -> 8 fp16 values, the same arithmetic as dequant16_bias
__device__ __forceinline__ v8h dequant8_bias(const uint2& w, const _Float16* __restrict__ bias,
                                             float dq) {
  const v8h b0 = *reinterpret_cast<const v8h*>(bias);
  const float off = -128.f * dq;
  const uint32_t u0 = w.x ^ 0x80808080u, u1 = w.y ^ 0x80808080u;
  v8h x;
  x[0] = (_Float16)fmaf(ubyte_f32<0>(u0), dq, off);
  x[1] = (_Float16)fmaf(ubyte_f32<1>(u0), dq, off);
  x[2] = (_Float16)fmaf(ubyte_f32<2>(u0), dq, off);
  x[3] = (_Float16)fmaf(ubyte_f32<3>(u0), dq, off);
  x[4] = (_Float16)fmaf(ubyte_f32<0>(u1), dq, off);
  x[5] = (_Float16)fmaf(ubyte_f32<1>(u1), dq, off);
  x[6] = (_Float16)fmaf(ubyte_f32<2>(u1), dq, off);
  x[7] = (_Float16)fmaf(ubyte_f32<3>(u1), dq, off);
  return x + b0;
}

// float2int8 of four values packed into one word, bit for bit: floor(med3(y, -127, 127.5)) ==
// clamp(floor(y), -127, 127) for every float y, so one converting instruction per value
// floors, converts and writes its byte in place.
__device__ __forceinline__ uint32_t float2int8_pack4(float x0, float x1, float x2, float x3,
                                                     float quant_scale) {
#pragma clang fp contract(off)
  const float y0 = __builtin_amdgcn_fmed3f(x0 * quant_scale + 0.5f, -127.f, 127.5f);
  const float y1 = __builtin_amdgcn_fmed3f(x1 * quant_scale + 0.5f, -127.f, 127.5f);
  const float y2 = __builtin_amdgcn_fmed3f(x2 * quant_scale + 0.5f, -127.f, 127.5f);
  const float y3 = __builtin_amdgcn_fmed3f(x3 * quant_scale + 0.5f, -127.f, 127.5f);
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


// ---------------------------------------------------------------------------------
// Attention of 32 queries per wavefront over one block of up to 128 keys staged in LDS:
// Ks row-major [128][D + 8] fp16 and Vt transposed [D][128 + 4] fp16 (rows of keys that do not
// exist are zero).  Scores are computed transposed (S^T = K Q^T) with
// v_mfma_f32_32x32x16_f16, so that lane (l32, g) owns query l32 of the wavefront and the keys
// sb * 32 + 8 * (i / 4) + 4 * g + (i % 4); the row maximum and sum need one cross-lane
// exchange, and the probability registers feed the P V product directly as its B operand.
// The rounding points are the reference's: scores and probabilities are rounded to fp16,
// the context is rounded to fp16 before it is quantised.
//
// All key fragments are requested from LDS before the first product and the products of the
// four blocks of 32 keys are interleaved, so neither the LDS latency nor the dependence
// between the products of one block is waited for; the value fragments are requested before
// the quotients are formed.  Padding costs no vector instruction per score: one more product
// per block adds -65504 * 65504 to the scores of the padded keys (contraction slot 0 of the
// lane half that holds the key's flag: lane g * 32 + l32 owns the flags of keys g * 32 + l32
// (padk0) and 64 + g * 32 + l32 (padk1)), which the conversion to fp16 turns into -inf as
// the mask would; all other scores receive +0.
//
// NKB: how many blocks of 32 keys exist (keys from NKB * 32 on are padding and are not looked
// at: a masked key's probability is exactly zero, so leaving its block out changes nothing).
// qreg[ks]: d = ks * 16 + g * 8 .. + 8 of the lane's query.  q_pad: the query is padding (its
// context is zero).  out_h / out_q: where the D context values of the lane's query go (fp16 /
// int8 codes), or null; nothing is stored when `live` is false.
constexpr int attn_kstr(int D) { return D + 8; }  // halfs per K row in LDS
constexpr int kAttnVstr = 128 + 4;                // halfs per V^T row in LDS

template <int D, int NKB = 4>
__device__ __forceinline__ void attend_block128(const _Float16* Ks, const _Float16* Vt,
                                                const v8h (&qreg)[D / 16], bool padk0, bool padk1,
                                                bool q_pad, bool live, float alpha,
                                                float quant_scale, __half* out_h, int8_t* out_q,
                                                int l32, int g) {
  constexpr int KSTR = attn_kstr(D), VSTR = kAttnVstr;
  v16f sc[NKB];
  {
    v8h kf[NKB][D / 16];
#pragma unroll
    for (int sb = 0; sb < NKB; ++sb)
#pragma unroll
      for (int ks = 0; ks < D / 16; ++ks)
        kf[sb][ks] = *reinterpret_cast<const v8h*>(&Ks[(sb * 32 + l32) * KSTR + ks * 16 + g * 8]);
    v8h bx = (v8h)(_Float16)0, ax[NKB];
    bx[0] = (_Float16)65504.f;
#pragma unroll
    for (int sb = 0; sb < NKB; ++sb) {
      ax[sb] = (v8h)(_Float16)0;
      ax[sb][0] = (g == (sb & 1) && (sb < 2 ? padk0 : padk1)) ? (_Float16)-65504.f : (_Float16)0;
    }
    __builtin_amdgcn_sched_barrier(0);
    v16f c[NKB];
#pragma unroll
    for (int sb = 0; sb < NKB; ++sb)
#pragma unroll
      for (int i = 0; i < 16; ++i) c[sb][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
#pragma unroll
      for (int sb = 0; sb < NKB; ++sb)
        c[sb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[sb][ks], qreg[ks], c[sb], 0, 0, 0);
#pragma unroll
    for (int sb = 0; sb < NKB; ++sb)
      c[sb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ax[sb], bx, c[sb], 0, 0, 0);
#pragma unroll
    for (int sb = 0; sb < NKB; ++sb)
#pragma unroll
      for (int i = 0; i < 16; ++i) sc[sb][i] = round_h(alpha * c[sb][i]);
  }

  // row maximum, exponentials (kept for the second pass) and their sum
  float m = kFloatInfNeg;
#pragma unroll
  for (int sb = 0; sb < NKB; ++sb)
#pragma unroll
    for (int i = 0; i < 16; ++i) m = fmaxf(m, sc[sb][i]);
  m = fmaxf(m, __shfl_xor(m, 32, 64));
  const float mref = m == kFloatInfNeg ? 0.f : m;
  const float nm = -mref * 1.44269504088896340736f;
  float sum = 0.f;
#pragma unroll
  for (int sb = 0; sb < NKB; ++sb)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      // exp(s - m) as 2^(s * log2(e) - m * log2(e)): one multiply-add and the exp2 instruction
      sc[sb][i] = __builtin_amdgcn_exp2f(fmaf(sc[sb][i], 1.44269504088896340736f, nm));
      sum += sc[sb][i];
    }
  sum += __shfl_xor(sum, 32, 64);

  // exp / sum is the correctly rounded quotient, as the reference's division gives:
  // exp * (1 / sum) differs from it by one unit in the last place often enough to flip fp16
  // probabilities, and a deep stack amplifies such flips.  The reciprocal is refined once per
  // query; one residual correction of the quotient then lands on the correctly rounded value
  // except within 2^-22 of a rounding boundary of the float quotient.
  float rs = __builtin_amdgcn_rcpf(sum);
  rs = sum > 0.f ? fmaf(fmaf(-sum, rs, 1.f), rs, rs) : 0.f;  // no visible key: all zero
  v16f acc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  v4h vf[NKB][2][D / 32][2];
#pragma unroll
  for (int sb = 0; sb < NKB; ++sb)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const _Float16* vrow = &Vt[(db * 32 + l32) * VSTR + sb * 32 + 16 * t + 4 * g];
        vf[sb][t][db][0] = *reinterpret_cast<const v4h*>(vrow);
        vf[sb][t][db][1] = *reinterpret_cast<const v4h*>(vrow + 8);
      }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int sb = 0; sb < NKB; ++sb) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      v8h pb;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float e = sc[sb][8 * t + j];
        float qt = e * rs;
        qt = fmaf(fmaf(-sum, qt, e), rs, qt);
        // keep the float quotient a value of its own: folded into the correction, the
        // conversion to fp16 would round once instead of twice
        asm volatile("" : "+v"(qt));
        pb[j] = (_Float16)qt;
      }
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const v4h lo = vf[sb][t][db][0], hi = vf[sb][t][db][1];
        const v8h a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb, acc[db], 0, 0, 0);
      }
    }
  }

  if (!live) return;
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
#pragma unroll
    for (int vg = 0; vg < 4; ++vg) {
      const int dd = db * 32 + 8 * vg + 4 * g;
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = round_h(acc[db][4 * vg + j]);
      if (out_h != nullptr) {
        half4_t t;
#pragma unroll
        for (int j = 0; j < 4; ++j) t.v[j] = __float2half_rn(q_pad ? 0.f : o[j]);
        *reinterpret_cast<half4_t*>(out_h + dd) = t;
      }
      if (out_q != nullptr) {
        // a padded query gives zeros, whose code is 0
        const uint32_t w4 = float2int8_pack4(o[0], o[1], o[2], o[3], quant_scale);
        *reinterpret_cast<uint32_t*>(out_q + dd) = q_pad ? 0u : w4;
      }
    }
  }
}

}  // namespace lsh
