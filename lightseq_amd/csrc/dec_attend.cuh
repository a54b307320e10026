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
#include "ls_device.cuh"

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
  return (long)((step_num + 63) & ~63) + 16 + NWV * D;
}

// q: the D query codes; kb / vb: the pair's cache rows [max_step][D]; out: where the D context
// codes go (nothing is stored unless `live`).  lds: decself_group_floats() floats of the group.
// wid: wavefront within the group, lane: lane within the wavefront.
template <int D, int NWV, int UN>
__device__ __forceinline__ void decself_attend_row(const int8_t* q, const int8_t* kb,
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

}  // namespace lsh
