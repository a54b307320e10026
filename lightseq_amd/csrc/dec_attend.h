// Decode-step self attention of one (row, head) pair over its int8 K/V cache by a group of NWV
// wavefronts: the body shared by the stand-alone kernel (one group per workgroup) and the
// kernel that computes the QKV projection first (several groups per workgroup).
//
// A cached key or value row of D bytes is read by D/16 adjacent lanes with one 16-byte load
// each, so a wavefront covers 1024 contiguous bytes of cache per load instruction and every
// byte of the cache is read once.  Scores are exact int32 dot products (v_dot4), probabilities
// live in LDS, the value sum is accumulated per lane over its share of the steps and then
// reduced across lanes (shuffles) and wavefronts (LDS) in a fixed tree.
// (inference/kernels/transformerKernels_int8.cc.cu:1515-1594 with the q.K product of
// model/quant_decoder.cc.cu:679-685 in front.)
#pragma once
#include "ls_device.h"

namespace lsh {

// Reductions over the NWV wavefronts of a group through the group's own `red` array.  Every
// thread of the workgroup reaches the barriers (all groups run the same code on the same
// step count).
template <int NWV>
__device__ __forceinline__ float group_sum(float v, float* red, int wid, int lane) {
  v = wave_sum(v);
  __syncthreads();  // protect `red` from a previous use
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < NWV; ++i) r += red[i];
  return r;
}
template <int NWV>
__device__ __forceinline__ float group_max(float v, float* red, int wid, int lane) {
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int i = 1; i < NWV; ++i) r = fmaxf(r, red[i]);
  return r;
}

// floats of LDS one group needs for a cache of `step_num` steps
template <int D, int NWV>
__host__ __device__ constexpr long decself_group_floats(int step_num) {
  const long rounds = (long)((step_num + 63) & ~63) + 16 + NWV * D;  // probabilities in LDS
  const long one = 32 + 4L * NWV * D;  // register-resident probabilities: four partials per wavefront
  return rounds > one ? rounds : one;
}

// q: the D query codes; kb / vb: the pair's cache rows [max_step][D]; out: where the D context
// codes go (nothing is stored unless `live`).  lds: decself_group_floats() floats of the group.
// wid: wavefront within the group, lane: lane within the wavefront.
template <int D, int NWV, int UN>
__device__ __forceinline__ void decself_attend_row_rounds(const int8_t* q, const int8_t* kb,
                                                          const int8_t* vb, int8_t* out, bool live,
                                                   int step_num, float attn_scale, float dq,
                                                   float quant_scale, float* lds, int wid,
                                                   int lane) {
#pragma clang fp contract(off)
  constexpr int CH = D / 16;    // lanes per cache row
  constexpr int KPW = 64 / CH;  // rows per wavefront per load
  const int padded = (step_num + 63) & ~63;
  float* probs = lds;           // [padded]
  float* red = lds + padded;    // [16] group reductions
  float* part = red + 16;       // [NWV][D] per-wavefront value sums
  const int tid = wid * 64 + lane;
  const int c = lane % CH, grp = lane / CH;
  const uint4 qv = *reinterpret_cast<const uint4*>(q + c * 16);

  // The cache is read in rounds of UN independent 16-byte loads per lane (UN * NWV * KPW
  // steps per round), all issued before the first is used: a step costs one memory round
  // trip per round instead of one per KPW * 4 cached steps.

  // scores -> scaled logits in LDS
  float mx = kFloatInfNeg;
  uint4 vv0[UN];
  for (int base = wid * KPW; base < step_num; base += UN * NWV * KPW) {
    uint4 kv[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int j = base + u * NWV * KPW + grp;
      // clamped instead of predicated: unconditional loads stay back to back
      kv[u] = *reinterpret_cast<const uint4*>(kb + (long)min(j, step_num - 1) * D + c * 16);
    }
    // The first round of value loads is requested right behind the first round of keys, before
    // any key is used: the two memory round trips of a short cache run side by side instead of
    // one after the other.
    if (base == wid * KPW) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int j = wid * KPW + u * NWV * KPW + grp;
        vv0[u] = *reinterpret_cast<const uint4*>(vb + (long)min(j, step_num - 1) * D + c * 16);
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int j = base + u * NWV * KPW + grp;
      int sc = 0;
      sc = __builtin_amdgcn_sdot4((int)qv.x, (int)kv[u].x, sc, false);
      sc = __builtin_amdgcn_sdot4((int)qv.y, (int)kv[u].y, sc, false);
      sc = __builtin_amdgcn_sdot4((int)qv.z, (int)kv[u].z, sc, false);
      sc = __builtin_amdgcn_sdot4((int)qv.w, (int)kv[u].w, sc, false);
#pragma unroll
      for (int m = 1; m < CH; m <<= 1) sc += __shfl_xor(sc, m, 64);
      if (j < step_num) {
        const float val = (float)sc * dq * dq * attn_scale;
        if (c == 0) probs[j] = val;
        mx = fmaxf(mx, val);
      }
    }
  }
  mx = group_max<NWV>(mx, red, wid, lane);
  float sum = 0.f;
  for (int j = tid; j < step_num; j += 64 * NWV) {
    const float e = __expf(probs[j] - mx);
    probs[j] = e;
    sum += e;
  }
  sum = group_sum<NWV>(sum, red, wid, lane);
  for (int j = tid; j < step_num; j += 64 * NWV) probs[j] = probs[j] / sum;
  __syncthreads();

  // value sum: lane (grp, c) accumulates dims [16c, 16c+16) over steps grp, grp + KPW * NWV, ...
  float acc[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) acc[k] = 0.f;
  for (int base = wid * KPW; base < step_num; base += UN * NWV * KPW) {
    uint4 vv[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int j = base + u * NWV * KPW + grp;
      if (base == wid * KPW)
        vv[u] = vv0[u];
      else
        vv[u] = *reinterpret_cast<const uint4*>(vb + (long)min(j, step_num - 1) * D + c * 16);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int j = base + u * NWV * KPW + grp;
      if (j < step_num) {  // same ascending order of steps per lane as a plain loop
        const float p = probs[j];
        const uint32_t w[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w};
#pragma unroll
        for (int k = 0; k < 16; ++k) acc[k] += (float)unpack_i8(w[k >> 2], k & 3) * p * dq;
      }
    }
  }
#pragma unroll
  for (int m = CH; m < 64; m <<= 1)
#pragma unroll
    for (int k = 0; k < 16; ++k) acc[k] += __shfl_xor(acc[k], m, 64);
  if (grp == 0) {
#pragma unroll
    for (int k = 0; k < 16; ++k) part[wid * D + c * 16 + k] = acc[k];
  }
  __syncthreads();
  if (tid < D) {
    float t[NWV];  // pairwise tree over the wavefronts' partial sums
#pragma unroll
    for (int i = 0; i < NWV; ++i) t[i] = part[i * D + tid];
#pragma unroll
    for (int st = 1; st < NWV; st *= 2)
#pragma unroll
      for (int i = 0; i < NWV; i += 2 * st) t[i] += t[i + st];
    if (live) out[tid] = (int8_t)float2int8(t[0], quant_scale);
  }
}

// ---- one round: the whole cache fits the UN loads of the group's lanes ----------------------
// A lane's scores never leave its registers: the 16 / CH-lane shuffle leaves every lane of a
// row group with the row's score, and the value loop walks the rows in the same lane order, so
// the probability a lane multiplies its value row with is the one it computed itself.  What is
// left of the softmax is two scalars per group (maximum, sum), exchanged through LDS with one
// barrier each; sums over the lanes of a wavefront use DPP row rotations and lane reads, no
// LDS permutes.  Dead slots (beyond the cache) carry probability zero and a clamped value row.

// v + v rotated by `n` lanes within each row of 16 lanes
template <int N>
__device__ __forceinline__ float row_ror_add(float v) {
  const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xf, 0xf, false);
  return v + __builtin_bit_cast(float, r);
}
template <int N>
__device__ __forceinline__ float row_ror_max(float v) {
  const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xf, 0xf, false);
  return fmaxf(v, __builtin_bit_cast(float, r));
}
__device__ __forceinline__ float lane_of(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
// int8 byte I of a word as float, one instruction
template <int I>
__device__ __forceinline__ float byte_to_float(uint32_t w) {
  float f;
  if (I == 0) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(f) : "v"(w));
  if (I == 1) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(f) : "v"(w));
  if (I == 2) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(f) : "v"(w));
  if (I == 3) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(f) : "v"(w));
  return f;
}

template <int D, int NWV, int UN>
__device__ __forceinline__ void decself_attend_row_once_body(uint4 qv, const uint4 (&kv)[UN],
                                                             const uint4 (&vv)[UN], int8_t* out,
                                                             bool live, int step_num,
                                                             float attn_scale, float dq,
                                                             float quant_scale, float* lds, int wid,
                                                             int lane);

// The cache rows of a lane for the register-resident form: lane (grp, c) of wavefront wid holds
// bytes [16 c, 16 c + 16) of rows (u NWV + wid) KPW + grp, u < UN (clamped to the last row,
// not predicated: unconditional loads stay back to back).
template <int D, int NWV, int UN>
__device__ __forceinline__ void decself_attend_load_rows(const int8_t* kb, const int8_t* vb,
                                                         int step_num, int wid, int lane,
                                                         uint4 (&kv)[UN], uint4 (&vv)[UN]) {
  constexpr int CH = D / 16, KPW = 64 / CH;
  const int c = lane % CH, grp = lane / CH;
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const int j = (u * NWV + wid) * KPW + grp;
    kv[u] = *reinterpret_cast<const uint4*>(kb + (long)min(j, step_num - 1) * D + c * 16);
  }
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const int j = (u * NWV + wid) * KPW + grp;
    vv[u] = *reinterpret_cast<const uint4*>(vb + (long)min(j, step_num - 1) * D + c * 16);
  }
}

template <int D, int NWV, int UN>
__device__ __forceinline__ void decself_attend_row_once(const int8_t* q, const int8_t* kb,
                                                        const int8_t* vb, int8_t* out, bool live,
                                                        int step_num, float attn_scale, float dq,
                                                        float quant_scale, float* lds, int wid,
                                                        int lane) {
  constexpr int CH = D / 16;
  const uint4 qv = *reinterpret_cast<const uint4*>(q + (lane % CH) * 16);
  uint4 kv[UN], vv[UN];
  decself_attend_load_rows<D, NWV, UN>(kb, vb, step_num, wid, lane, kv, vv);
  decself_attend_row_once_body<D, NWV, UN>(qv, kv, vv, out, live, step_num, attn_scale, dq,
                                           quant_scale, lds, wid, lane);
}

// What follows the loads: scores, soft-max, value sums, the context codes.  The fused
// projection + attention kernel requests the rows before its product and enters here.
template <int D, int NWV, int UN>
__device__ __forceinline__ void decself_attend_row_once_body(uint4 qv, const uint4 (&kv)[UN],
                                                             const uint4 (&vv)[UN], int8_t* out,
                                                             bool live, int step_num,
                                                             float attn_scale, float dq,
                                                             float quant_scale, float* lds, int wid,
                                                             int lane) {
#pragma clang fp contract(off)
  constexpr int CH = D / 16;    // lanes per cache row
  constexpr int KPW = 64 / CH;  // rows per wavefront per load
  float* red_max = lds;         // [NWV]
  float* red_sum = lds + 16;    // [NWV]
  float* part = lds + 32;       // [NWV * 4][D] value sums per row of 16 lanes
  const int c = lane % CH, grp = lane / CH;
  // scores of the lane's rows (every lane of a row group ends with the row's score)
  float val[UN];
  float mx = kFloatInfNeg;
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const int j = (u * NWV + wid) * KPW + grp;
    int sc = 0;
    sc = __builtin_amdgcn_sdot4((int)qv.x, (int)kv[u].x, sc, false);
    sc = __builtin_amdgcn_sdot4((int)qv.y, (int)kv[u].y, sc, false);
    sc = __builtin_amdgcn_sdot4((int)qv.z, (int)kv[u].z, sc, false);
    sc = __builtin_amdgcn_sdot4((int)qv.w, (int)kv[u].w, sc, false);
    // the CH partial dot products of the row: lanes l ^ 1, l ^ 2 by quad permutation
    if (CH >= 2) sc += __builtin_amdgcn_update_dpp(0, sc, 0xB1, 0xf, 0xf, false);
    if (CH >= 4) sc += __builtin_amdgcn_update_dpp(0, sc, 0x4E, 0xf, 0xf, false);
    if (CH >= 8) sc += __shfl_xor(sc, 4, 64);
    val[u] = j < step_num ? (float)sc * dq * dq * attn_scale : kFloatInfNeg;
    mx = fmaxf(mx, val[u]);
  }
  // maximum over the group: rows of 16 lanes, the four rows of the wavefront, the wavefronts
  mx = row_ror_max<8>(row_ror_max<4>(row_ror_max<2>(row_ror_max<1>(mx))));
  mx = fmaxf(fmaxf(lane_of(mx, 0), lane_of(mx, 16)), fmaxf(lane_of(mx, 32), lane_of(mx, 48)));
  if (lane == 0) red_max[wid] = mx;
  __syncthreads();
  mx = red_max[0];
#pragma unroll
  for (int i = 1; i < NWV; ++i) mx = fmaxf(mx, red_max[i]);
  // exp and the sum over the group (every row once: lanes of one c, rotations by multiples of CH)
  float sum = 0.f;
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const int j = (u * NWV + wid) * KPW + grp;
    val[u] = j < step_num ? __expf(val[u] - mx) : 0.f;
    sum += val[u];
  }
  if (CH <= 1) sum = row_ror_add<1>(sum);
  if (CH <= 2) sum = row_ror_add<2>(sum);
  if (CH <= 4) sum = row_ror_add<4>(sum);
  sum = row_ror_add<8>(sum);
  sum = (lane_of(sum, 0) + lane_of(sum, 16)) + (lane_of(sum, 32) + lane_of(sum, 48));
  if (lane == 0) red_sum[wid] = sum;
  __syncthreads();
  sum = red_sum[0];
#pragma unroll
  for (int i = 1; i < NWV; ++i) sum += red_sum[i];
  // value sum: lane (grp, c) accumulates dims [16c, 16c+16) over its rows, in ascending order
  float acc[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) acc[k] = 0.f;
#pragma unroll
  for (int u = 0; u < UN; ++u) {
    const float pd = val[u] / sum * dq;
    const uint32_t w[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w};
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      acc[4 * q4 + 0] = __builtin_fmaf(byte_to_float<0>(w[q4]), pd, acc[4 * q4 + 0]);
      acc[4 * q4 + 1] = __builtin_fmaf(byte_to_float<1>(w[q4]), pd, acc[4 * q4 + 1]);
      acc[4 * q4 + 2] = __builtin_fmaf(byte_to_float<2>(w[q4]), pd, acc[4 * q4 + 2]);
      acc[4 * q4 + 3] = __builtin_fmaf(byte_to_float<3>(w[q4]), pd, acc[4 * q4 + 3]);
    }
  }
  // rows of 16 lanes by rotation, then the 4 NWV row sums through LDS
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    if (CH <= 1) acc[k] = row_ror_add<1>(acc[k]);
    if (CH <= 2) acc[k] = row_ror_add<2>(acc[k]);
    if (CH <= 4) acc[k] = row_ror_add<4>(acc[k]);
    acc[k] = row_ror_add<8>(acc[k]);
  }
  if ((lane & 15) < CH) {
    float* p = part + (wid * 4 + (lane >> 4)) * D + c * 16;
#pragma unroll
    for (int k = 0; k < 16; k += 4)
      *reinterpret_cast<float4*>(p + k) = make_float4(acc[k], acc[k + 1], acc[k + 2], acc[k + 3]);
  }
  __syncthreads();
  const int tid = wid * 64 + lane;
  if (tid < D) {
    float t[4 * NWV];  // pairwise tree over the partial sums
#pragma unroll
    for (int i = 0; i < 4 * NWV; ++i) t[i] = part[i * D + tid];
#pragma unroll
    for (int st = 1; st < 4 * NWV; st *= 2)
#pragma unroll
      for (int i = 0; i < 4 * NWV; i += 2 * st) t[i] += t[i + st];
    if (live) out[tid] = (int8_t)float2int8(t[0], quant_scale);
  }
}

// The group's attention: one round where the cache fits it, otherwise rounds through LDS.  The
// choice follows the cache length only, so a row's result does not depend on its batch.
template <int D, int NWV, int UN>
__device__ __forceinline__ void decself_attend_row(const int8_t* q, const int8_t* kb,
                                                   const int8_t* vb, int8_t* out, bool live,
                                                   int step_num, float attn_scale, float dq,
                                                   float quant_scale, float* lds, int wid,
                                                   int lane) {
  if (step_num <= UN * NWV * (64 / (D / 16)))
    decself_attend_row_once<D, NWV, UN>(q, kb, vb, out, live, step_num, attn_scale, dq,
                                        quant_scale, lds, wid, lane);
  else
    decself_attend_row_rounds<D, NWV, UN>(q, kb, vb, out, live, step_num, attn_scale, dq,
                                          quant_scale, lds, wid, lane);
}

}  // namespace lsh
