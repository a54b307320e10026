// LayerNorm family of the int8 layer path: dequant + residual (+colsum) +
// LayerNorm + quant, one HBM pass.
//
// Two layouts, both keeping a token row in registers with the reference's two-pass mean
// and variance reduced by cross-lane shuffles:
//  * ln_rows8_kernel (hidden % 8 == 0): a row belongs to LPR lanes (32: two rows per
//    wavefront), 8 consecutive elements per lane per step (16-byte fp16, 32-byte int32
//    accesses); scale, bias and residual bias are fetched with the first round of loads;
//    with nparts > 1 the int32 input is the exact integer sum of nparts split-K
//    accumulator planes, loaded independently.
//  * ln_rows_kernel (any hidden): one wavefront per row, 4 elements per lane per step.
//
// Replaces inference/kernels/transformerKernels_int8.cc.cu:149-863.
#include "ls_device.h"
#include "ls_launch.h"
#include "ln_rows8.h"

#include <hip/hip_ext.h>

#include <type_traits>

namespace lsh {


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

template <typename T, typename AccT, int MODE, int LPR, int ITER>
__global__ void __launch_bounds__(256)
ln_rows8_kernel(const AccT* __restrict__ gemm_out, T* residual, T* out_t,
                int8_t* __restrict__ out_q, const T* __restrict__ scale,
                const T* __restrict__ bias, const T* __restrict__ residual_bias,
                const T* __restrict__ colsum, int tokens, int hidden, float dequant_scale,
                float quant_scale, int is_post_ln, int nparts, long part_stride) {
  constexpr int RPW = kWave / LPR;
  const int lane = threadIdx.x & 63;
  const int row = (blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW + lane / LPR;
  // dead rows keep the shuffles convergent
  ln_rows8_row<T, AccT, MODE, LPR, ITER>(row, row < tokens, lane % LPR, gemm_out, residual, out_t,
                                         out_q, scale, bias, residual_bias, colsum, hidden,
                                         dequant_scale, quant_scale, is_post_ln, nparts,
                                         part_stride);
}

// ---------------------------------------------------------------------------------
// Out-projection GEMM + dequant + residual + LayerNorm + quant in one kernel, for products
// whose output is one hidden-size-wide row per token (N = K = hidden in {512, 768, 1024}).
// Replaces the pair cublasLtMM_withAlgo_i8IO + ker_residual_bias_ln_i8I_i8O
// (inference/model/quant_bert_encoder.cc.cu:361-396) with the same rounding points -- the
// product is requantised to its int8 code first, then dequantised, added to the residual and
// normalised -- and the very row routine of the stand-alone kernel, so the two routes give
// the same bytes.
//
// A workgroup owns 16 token rows and all N columns: 8 wavefronts x NT 16-column blocks,
// v_mfma_i32_16x16x64_i8 with the weight block as the row operand.  The 16 x K activation
// panel and the weights are read straight into MFMA registers, three K slices in flight, the
// weights from a copy tiled at load time so that a wavefront's fragment is 1 KB contiguous.  Nothing goes through LDS but the
// 16 x N tile of int8 codes handed to the row routine (two rows per wavefront, as it expects).
// Every workgroup streams the whole weight matrix (it stays in the XCD's L2), which is what
// bounds the kernel: N * K bytes per compute unit at ~64 B/clk.
// ---------------------------------------------------------------------------------
typedef int ln_v4i __attribute__((ext_vector_type(4)));

// [N, K] int8 row-major -> blocks of 16 rows x 64 bytes in MFMA lane order:
// tiled[((n / 16) * (K / 64) + k / 64) * 1024 + lane * 16 + b] with lane = (k % 64) / 16 * 16 + n % 16
__global__ void __launch_bounds__(256)
tile_weight_16x64_kernel(const int8_t* __restrict__ w, int8_t* __restrict__ tiled, int N, int K) {
  const long chunk = (long)blockIdx.x * 256 + threadIdx.x;  // one 16-byte chunk each
  const long total = (long)N * K / 16;
  if (chunk >= total) return;
  const int lane = (int)(chunk & 63);
  const long blk = chunk >> 6;
  const int ks = (int)(blk % (K / 64)), nt = (int)(blk / (K / 64));
  const int n = nt * 16 + (lane & 15), k = ks * 64 + (lane >> 4) * 16;
  *reinterpret_cast<ln_v4i*>(tiled + chunk * 16) =
      *reinterpret_cast<const ln_v4i*>(w + (long)n * K + k);
}

template <typename T, int NT, int KS, int LPR, int ITER>
__global__ void __launch_bounds__(512)
gemm_ln_rows16_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ Wt, float alpha,
                      T* residual, int8_t* __restrict__ out_q, const T* __restrict__ scale,
                      const T* __restrict__ bias, const T* __restrict__ residual_bias, int tokens,
                      float dequant_scale, float quant_scale, int is_post_ln) {
  constexpr int N = 8 * NT * 16, K = KS * 64;
  __shared__ __align__(16) int8_t codes[16 * N];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r0 = blockIdx.x * 16;
  // The K slices are walked from a starting slice that differs between the workgroups of an
  // XCD (workgroup b runs on XCD b % 8), wrapping around: integer sums commute, and workgroups
  // that all stream the same weight matrix in the same order at the same time would queue up
  // on the same L2 channel.
  const int rot = ((int)blockIdx.x >> 3) % KS;
  // activation fragments: row r0 + lane % 16 (clamped: rows beyond the tensor are never stored)
  const int8_t* ap = A + (long)min(r0 + (lane & 15), tokens - 1) * K + (lane >> 4) * 16;
  // weight fragments of this wavefront's NT column blocks
  const int8_t* wp = Wt + ((long)wave * NT * KS * 64 + lane) * 16;
  ln_v4i wf[3][NT], af[3];
  auto load_slice = [&](int i) {  // i-th slice of this workgroup's walk, into ring slot i % 3
    int ks = i + rot;
    if (ks >= KS) ks -= KS;
    af[i % 3] = *reinterpret_cast<const ln_v4i*>(ap + ks * 64);
#pragma unroll
    for (int t = 0; t < NT; ++t)
      wf[i % 3][t] = *reinterpret_cast<const ln_v4i*>(wp + ((long)t * KS + ks) * 1024);
  };
  ln_v4i acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = (ln_v4i)0;
  // the residual rows the layer norm will add are requested now, so that they have arrived
  // when the product is done (same lane layout as the row routine below)
  constexpr int RPW = kWave / LPR, PASSES = 16 / (8 * RPW);
  half8_t pre[PASSES][ITER];
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const int row = min(r0 + (pass * 8 + wave) * RPW + lane / LPR, tokens - 1);
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int e = min((it * LPR + lane % LPR) * 8, N - 8);
        pre[pass][it] = *reinterpret_cast<const half8_t*>(
            reinterpret_cast<const __half*>(residual) + (long)row * N + e);
      }
    }
  }
  load_slice(0);
  if (KS > 1) load_slice(1);
  // the scheduling barriers keep the loads of slice i + 2 ahead of the MFMAs of slice i:
  // left alone, the compiler sinks every load to just before its use and the loop waits for
  // memory at each step
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < KS; ++i) {
    if (i + 2 < KS) load_slice(i + 2);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NT; ++t)
      acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[i % 3][t], af[i % 3], acc[t], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  // lane holds C[token lane % 16][column block * 16 + 4 * (lane / 16) + 0..3]
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = (wave * NT + t) * 16 + 4 * (lane >> 4);
    *reinterpret_cast<uint32_t*>(codes + (lane & 15) * N + n) =
        requant_acc_pack4(acc[t][0], acc[t][1], acc[t][2], acc[t][3], alpha);
  }
  __syncthreads();
  // the stand-alone kernel's row routine with the lane layout it uses for this hidden size
  // (LPR lanes per row), fed from the staged codes
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int row = r0 + (pass * 8 + wave) * RPW + lane / LPR;
    ln_rows8_row<T, int8_t, kLnResQuant, LPR, ITER>(
        row, row < tokens, lane % LPR, codes - (long)r0 * N, residual, nullptr, out_q, scale, bias,
        residual_bias, nullptr, N, dequant_scale, quant_scale, is_post_ln, 1, 0,
        sizeof(T) == 2 ? pre[pass] : nullptr, r0);
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

// What follows the row's values in the workgroup-per-row kernels: mean, variance, the
// normalised row, its int8 codes and the new residual stream.  x: the lane's four values (0
// beyond the row), on: the lane holds elements of the row.
template <typename T, int MODE>
__device__ __forceinline__ void
ln_row_wg_finish(const float (&x)[4], bool on, int e, long base, const float (&g)[4],
                 const float (&b)[4], const float (&rb)[4], T* residual, T* out_t,
                 int8_t* __restrict__ out_q, int hidden, float quant_scale, int is_post_ln,
                 float (*red)[4]) {
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wpr = (int)blockDim.x >> 6;  // wavefronts of the row
  auto row_total = [&](float v, float* r) {
    v = wave_sum_dpp(v);
    if (lane == 0) r[wid] = v;
    __syncthreads();
    // ascending order, without a loop (wpr <= 4)
    float t = r[0];
    const float r1 = r[1], r2 = r[2], r3 = r[3];
    if (wpr > 1) t += r1;
    if (wpr > 2) t += r2;
    if (wpr > 3) t += r3;
    return t;
  };
  const float mean = row_total((x[0] + x[1]) + (x[2] + x[3]), red[0]) / (float)hidden;
  float var = 0.f;
  if (on) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float t = x[k] - mean;
      var += t * t;
    }
  }
  const float rstd = rsqrtf(row_total(var, red[1]) / (float)hidden + kLnEpsilon);
  if (!on) return;
  float o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = (x[k] - mean) * rstd * TT<T>::safe(g[k]) + TT<T>::safe(b[k]);
  if (MODE == kLnResOut) {
    st4(out_t, base + e, o);
  } else {
    *reinterpret_cast<uint32_t*>(out_q + base + e) =
        pack4_i8(float2int8(o[0], quant_scale), float2int8(o[1], quant_scale),
                 float2int8(o[2], quant_scale), float2int8(o[3], quant_scale));
    float w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float keep = is_post_ln ? o[k] : x[k];
      w[k] = (MODE == kLnFirst) ? keep + rb[k] : TT<T>::rnd(keep) + rb[k];
    }
    st4(residual, base + e, w);
  }
}

// One row per workgroup, 4 consecutive elements per lane (hidden <= 4 * blockDim.x, hidden
// % 4 == 0): the layer norm of the decode steps, where a launch lasts a few microseconds and
// every dependent step inside it shows.  So: no integer division and no branch before the loads
// (indices are clamped, not predicated, which also lets the kernel arguments arrive in one
// batch), every load -- parameters and up to four accumulator planes -- requested before the
// first is used, sums over a wavefront by DPP permutations and lane reads instead of LDS
// permutes, and one barrier per reduction.
// Order of a row sum: (x0 + x1) + (x2 + x3) per lane; lanes of a quad, the quads of a row of
// 16 lanes and the four rows of a wavefront pairwise; the wavefronts in ascending order.
template <typename T, typename AccT, int MODE>
__global__ void __launch_bounds__(256)
ln_row_wg_kernel(const AccT* __restrict__ gemm_out, T* residual, T* out_t,
                 int8_t* __restrict__ out_q, const T* __restrict__ scale,
                 const T* __restrict__ bias, const T* __restrict__ residual_bias,
                 const T* __restrict__ colsum, int hidden, float dequant_scale,
                 float quant_scale, int is_post_ln, int nparts, long part_stride) {
  __shared__ float red[2][4];
  const int e0 = (int)threadIdx.x * 4;
  const bool on = e0 < hidden;
  const int e = on ? e0 : 0;  // lanes past the row load its first elements and drop them
  const long base = (long)blockIdx.x * hidden;
  float g[4], b[4], rb[4] = {0.f, 0.f, 0.f, 0.f}, r[4], c[4] = {0.f, 0.f, 0.f, 0.f};
  ld4(residual, base + e, r);
  // every load of the kernel is requested before the first value is used (the parameters
  // before the accumulator planes, whose sums wait for them); optional operands through a
  // pointer that is always valid, dropped afterwards: a load inside a branch is followed by
  // its wait, one memory round trip after the other
  const bool has_rb = MODE != kLnResOut && residual_bias != nullptr;
  const bool has_cs = MODE != kLnFirst && colsum != nullptr;
  auto g_raw = ld4_raw(scale, e), b_raw = ld4_raw(bias, e);
  auto rb_raw = ld4_raw(has_rb ? residual_bias : scale, e);
  auto c_raw = ld4_raw(has_cs ? colsum : scale, e);
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  if (MODE != kLnFirst) {
    if constexpr (sizeof(AccT) == 4) {
      // up to four planes in flight together (what the decode-step products write; integer
      // sums: any order gives the same bits); a plane index beyond the last is clamped for the
      // load and its value dropped
      int4 m[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        m[u] = *reinterpret_cast<const int4*>(gemm_out + (long)min(u, nparts - 1) * part_stride +
                                              base + e);
      pin4(g_raw, b_raw, rb_raw, c_raw);  // (requested ahead of the planes: they are here first)
#pragma unroll
      for (int u = 0; u < 4; ++u)
        asm volatile("" : "+v"(m[u].x), "+v"(m[u].y), "+v"(m[u].z), "+v"(m[u].w));
      int4 acc = m[0];
#pragma unroll
      for (int u = 1; u < 4; ++u) {
        const bool on_u = u < nparts;
        acc.x += on_u ? m[u].x : 0; acc.y += on_u ? m[u].y : 0;
        acc.z += on_u ? m[u].z : 0; acc.w += on_u ? m[u].w : 0;
      }
      for (int p = 4; p < nparts; ++p) {
        const int4 t = *reinterpret_cast<const int4*>(gemm_out + (long)p * part_stride + base + e);
        acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
      }
      a[0] = (float)acc.x; a[1] = (float)acc.y; a[2] = (float)acc.z; a[3] = (float)acc.w;
    } else {
      ld4_acc(gemm_out, base + e, a);
      pin4(g_raw, b_raw, rb_raw, c_raw);
    }
  } else {
    pin4(g_raw, b_raw, rb_raw, c_raw);
  }
  cvt4(g_raw, g);
  cvt4(b_raw, b);
  cvt4(rb_raw, rb);
  cvt4(c_raw, c);
#pragma unroll
  for (int k = 0; k < 4; ++k) rb[k] = has_rb ? rb[k] : 0.f;
  float x[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (MODE == kLnFirst) {
      x[k] = TT<T>::safe(r[k]);
    } else {
      x[k] = a[k] * dequant_scale + TT<T>::safe(r[k]);
      if (colsum != nullptr) x[k] += TT<T>::safe(c[k]);
    }
    if (!on) x[k] = 0.f;
  }
  ln_row_wg_finish<T, MODE>(x, on, e, base, g, b, rb, residual, out_t, out_q, hidden, quant_scale,
                            is_post_ln, red);
}

// The workgroup-per-row kernel is chosen by the caller, never by the row count: the two
// kernels add a row's elements in different orders, and a sequence's result must not depend
// on how many other rows share its launch.  The decode-step paths (a few rows per launch)
// select it for the duration of a step; everything else runs the 8-wide kernel.  Measured at
// hidden 768 / 1024: 3.3-4.7 us against 4.2-5.9 us up to 1024 rows, 8.6-10.9 us against
// 7.3-8.3 us at 4096 rows; more than one row per workgroup was slower at every size.
static thread_local bool g_ln_few_rows = false;
LnFewRowsScope::LnFewRowsScope() : _prev(g_ln_few_rows) { g_ln_few_rows = true; }
LnFewRowsScope::~LnFewRowsScope() { g_ln_few_rows = _prev; }
bool ln_set_few_rows(bool on) {
  const bool prev = g_ln_few_rows;
  g_ln_few_rows = on;
  return prev;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The decoder's target embedding (inference/kernels/embKernels_int8.cc.cu:158-200) and the first
// layer norm of the stack (ker_norm_layer_resual_i8O) in one launch, for the decode steps: a
// row's embedding -- int8 table row (vocabulary-major) * scale + position row, rounded to the
// storage type as the stand-alone kernel stores it -- is the row the layer norm reads, so the
// bytes are those of launch_dec_emb_i8I followed by ker_norm_layer_resual_i8O with the row
// kernel.  The token id is one dependent load ahead of the table row; the parameters travel
// meanwhile.
template <typename T>
__global__ void __launch_bounds__(256)
dec_emb_ln_row_wg_kernel(const int8_t* __restrict__ token_emb, const T* __restrict__ pos_emb,
                         const int* __restrict__ tokens, T* residual,
                         int8_t* __restrict__ out_q, const T* __restrict__ scale,
                         const T* __restrict__ bias, const T* __restrict__ residual_bias,
                         int hidden, int vocab, int step, int max_step, float emb_scale,
                         float quant_scale, int is_post_ln) {
#pragma clang fp contract(off)
  __shared__ float red[2][4];
  const int e0 = (int)threadIdx.x * 4;
  const bool on = e0 < hidden;
  const int e = on ? e0 : 0;
  const long base = (long)blockIdx.x * hidden;
  int token = tokens[(long)blockIdx.x * max_step + step];
  const bool has_rb = residual_bias != nullptr;
  auto g_raw = ld4_raw(scale, e), b_raw = ld4_raw(bias, e);
  auto rb_raw = ld4_raw(has_rb ? residual_bias : scale, e);
  auto p_raw = ld4_raw(pos_emb, (long)step * hidden + e);
  token = min(max(token, 0), vocab - 1);  // never index outside the table
  const uint32_t ew = *reinterpret_cast<const uint32_t*>(token_emb + (long)token * hidden + e);
  pin4(g_raw, b_raw, rb_raw, p_raw);
  float g[4], b[4], rb[4], pos[4], x[4];
  cvt4(g_raw, g);
  cvt4(b_raw, b);
  cvt4(rb_raw, rb);
  cvt4(p_raw, pos);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    rb[k] = has_rb ? rb[k] : 0.f;
    const float v = (float)unpack_i8(ew, k) * emb_scale + pos[k];
    x[k] = on ? TT<T>::safe(TT<T>::rnd(v)) : 0.f;
  }
  ln_row_wg_finish<T, kLnFirst>(x, on, e, base, g, b, rb, residual, nullptr, out_q, hidden,
                                quant_scale, is_post_ln, red);
}

template <typename T>
int dec_emb_norm_layer_i8O(const int8_t* token_emb, const T* pos_emb, const int* tokens,
                           T* residual, int8_t* out_q, const T* scale, const T* bias,
                           const T* residual_bias, int rows, int hidden, int vocab, int step,
                           int max_step, float dequant_scale, bool scaled, float quant_scale,
                           bool is_post_ln, hipStream_t s) {
  if (!token_emb || !pos_emb || !tokens || !residual || !out_q || !scale || !bias || rows <= 0 ||
      hidden <= 0 || vocab <= 0 || max_step <= 0)
    return lsh_fail(LSH_ERR_INVALID, "dec_emb_norm_layer_i8O: bad arguments");
  if (step < 0 || step >= max_step) return lsh_fail(LSH_ERR_INVALID, "violate step < max_step");
  if (hidden % 4 != 0 || hidden > 1024 || !aligned16(token_emb) || !aligned16(pos_emb) ||
      !aligned16(residual) || !aligned16(out_q) || !aligned16(scale) || !aligned16(bias) ||
      !aligned16(residual_bias))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "dec_emb_norm_layer_i8O: needs hidden % 4 == 0, hidden <= 1024, aligned operands");
  float emb_scale = dequant_scale;
  if (scaled) emb_scale *= sqrtf((float)hidden);
  const int tpr = ((hidden / 4 + 63) / 64) * 64;
  dec_emb_ln_row_wg_kernel<T><<<rows, tpr, 0, s>>>(token_emb, pos_emb, tokens, residual, out_q,
                                                   scale, bias, residual_bias, hidden, vocab, step,
                                                   max_step, emb_scale, quant_scale,
                                                   is_post_ln ? 1 : 0);
  return lsh_check_launch("dec_emb_ln_row_wg_kernel");
}
template int dec_emb_norm_layer_i8O<__half>(const int8_t*, const __half*, const int*, __half*,
                                            int8_t*, const __half*, const __half*, const __half*,
                                            int, int, int, int, int, float, bool, float, bool,
                                            hipStream_t);
template int dec_emb_norm_layer_i8O<float>(const int8_t*, const float*, const int*, float*,
                                           int8_t*, const float*, const float*, const float*, int,
                                           int, int, int, int, float, bool, float, bool,
                                           hipStream_t);

// The same for a generation step of the GPT model: the embedding of one token per sequence at
// position `pos` (a padding token gives zeros), the token counted into real_seq_len and
// zero_flag cleared as gpt_embedding_step_kernel does, then the first layer's layer norm.
template <typename T>
__global__ void __launch_bounds__(256)
gpt_emb_ln_row_wg_kernel(const int8_t* __restrict__ token_emb, const T* __restrict__ pos_emb,
                         const int* __restrict__ token_id, T* residual,
                         int8_t* __restrict__ out_q, const T* __restrict__ scale,
                         const T* __restrict__ bias, const T* __restrict__ residual_bias,
                         int* real_seq_len, int* zero_flag, int padding_id, int hidden, int vocab,
                         int pos, float emb_scale, float quant_scale, int is_post_ln) {
#pragma clang fp contract(off)
  __shared__ float red[2][4];
  const int e0 = (int)threadIdx.x * 4;
  const bool on = e0 < hidden;
  const int e = on ? e0 : 0;
  const long base = (long)blockIdx.x * hidden;
  int token = token_id[blockIdx.x];
  const bool has_rb = residual_bias != nullptr;
  auto g_raw = ld4_raw(scale, e), b_raw = ld4_raw(bias, e);
  auto rb_raw = ld4_raw(has_rb ? residual_bias : scale, e);
  auto p_raw = ld4_raw(pos_emb, (long)pos * hidden + e);
  const bool pad = token == padding_id;
  token = min(max(token, 0), vocab - 1);  // never index outside the table
  const uint32_t ew = *reinterpret_cast<const uint32_t*>(token_emb + (long)token * hidden + e);
  if (threadIdx.x == 0) {
    if (!pad) real_seq_len[blockIdx.x] += 1;
    if (zero_flag != nullptr && blockIdx.x == 0) zero_flag[0] = 0;
  }
  pin4(g_raw, b_raw, rb_raw, p_raw);
  float g[4], b[4], rb[4], pe[4], x[4];
  cvt4(g_raw, g);
  cvt4(b_raw, b);
  cvt4(rb_raw, rb);
  cvt4(p_raw, pe);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    rb[k] = has_rb ? rb[k] : 0.f;
    const float v = pad ? 0.f : (float)unpack_i8(ew, k) * emb_scale + pe[k];
    x[k] = on ? TT<T>::safe(TT<T>::rnd(v)) : 0.f;
  }
  ln_row_wg_finish<T, kLnFirst>(x, on, e, base, g, b, rb, residual, nullptr, out_q, hidden,
                                quant_scale, is_post_ln, red);
}

template <typename T>
int gpt_emb_step_norm_layer_i8O(const int8_t* token_emb, const T* pos_emb, const int* token_id,
                                T* residual, int8_t* out_q, const T* scale, const T* bias,
                                const T* residual_bias, int* real_seq_len, int* zero_flag,
                                int batch_size, int hidden, int vocab, int padding_id, int pos,
                                int max_step, float dequant_scale, float quant_scale,
                                bool is_post_ln, hipStream_t s) {
  if (!token_emb || !pos_emb || !token_id || !residual || !out_q || !scale || !bias ||
      !real_seq_len || batch_size <= 0 || hidden <= 0 || vocab <= 0)
    return lsh_fail(LSH_ERR_INVALID, "gpt_emb_step_norm_layer_i8O: bad arguments");
  if (pos < 0 || pos >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "gpt_emb_step_norm_layer_i8O: position outside the table");
  if (hidden % 4 != 0 || hidden > 1024 || !aligned16(token_emb) || !aligned16(pos_emb) ||
      !aligned16(residual) || !aligned16(out_q) || !aligned16(scale) || !aligned16(bias) ||
      !aligned16(residual_bias))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "gpt_emb_step_norm_layer_i8O: needs hidden % 4 == 0, hidden <= 1024, aligned "
                    "operands");
  const int tpr = ((hidden / 4 + 63) / 64) * 64;
  gpt_emb_ln_row_wg_kernel<T><<<batch_size, tpr, 0, s>>>(
      token_emb, pos_emb, token_id, residual, out_q, scale, bias, residual_bias, real_seq_len,
      zero_flag, padding_id, hidden, vocab, pos, dequant_scale, quant_scale, is_post_ln ? 1 : 0);
  return lsh_check_launch("gpt_emb_ln_row_wg_kernel");
}
template int gpt_emb_step_norm_layer_i8O<__half>(const int8_t*, const __half*, const int*,
                                                 __half*, int8_t*, const __half*, const __half*,
                                                 const __half*, int*, int*, int, int, int, int,
                                                 int, int, float, float, bool, hipStream_t);
template int gpt_emb_step_norm_layer_i8O<float>(const int8_t*, const float*, const int*, float*,
                                                int8_t*, const float*, const float*, const float*,
                                                int*, int*, int, int, int, int, int, int, float,
                                                float, bool, hipStream_t);

template <typename T, typename AccT, int MODE>
static int launch_ln(const AccT* gemm_out, T* residual, T* out_t, int8_t* out_q, const T* scale,
                     const T* bias, const T* residual_bias, const T* colsum, int tokens,
                     int hidden, float dequant_scale, float quant_scale, int is_post_ln,
                     hipStream_t stream, int nparts = 1, long part_stride = 0) {
  if (tokens <= 0 || hidden <= 0) return lsh_fail(LSH_ERR_INVALID, "layer norm: empty shape");
  if (nparts < 1 || (nparts > 1 && (sizeof(AccT) != 4 || part_stride % 4 != 0)))
    return lsh_fail(LSH_ERR_INVALID, "layer norm: bad accumulator planes");
  const bool vec_ok = hidden % 4 == 0 && hidden <= 2048 && aligned16(gemm_out) &&
                      aligned16(residual) && aligned16(out_t) && aligned16(out_q) &&
                      aligned16(scale) && aligned16(bias) && aligned16(residual_bias) &&
                      aligned16(colsum);
  if (vec_ok && hidden <= 1024 && g_ln_few_rows) {
    const int tpr = ((hidden / 4 + 63) / 64) * 64;  // threads of a row: whole wavefronts
    ln_row_wg_kernel<T, AccT, MODE><<<tokens, tpr, 0, stream>>>(
        gemm_out, residual, out_t, out_q, scale, bias, residual_bias, colsum, hidden,
        dequant_scale, quant_scale, is_post_ln, nparts, part_stride);
    return lsh_check_launch("ln_row_wg_kernel");
  }
  if (vec_ok && hidden % 8 == 0) {
    // LPR = 64 when the row fills whole 512-element steps, otherwise two rows per wavefront
#define LSH_LN8_CASE(LPR, IT)                                                                    \
  ln_rows8_kernel<T, AccT, MODE, LPR, IT>                                                        \
      <<<(tokens + 4 * (64 / LPR) - 1) / (4 * (64 / LPR)), 256, 0, stream>>>(                    \
          gemm_out, residual, out_t, out_q, scale, bias, residual_bias, colsum, tokens, hidden,  \
          dequant_scale, quant_scale, is_post_ln, nparts, part_stride)
    if (hidden <= 256) LSH_LN8_CASE(32, 1);
    else if (hidden <= 512) LSH_LN8_CASE(32, 2);
    else if (hidden <= 768) LSH_LN8_CASE(32, 3);
    else if (hidden <= 1024) LSH_LN8_CASE(64, 2);
    else if (hidden <= 1536) LSH_LN8_CASE(64, 3);
    else LSH_LN8_CASE(64, 4);
#undef LSH_LN8_CASE
    return lsh_check_launch("ln_rows8_kernel");
  }
  if (nparts > 1)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "layer norm: accumulator planes need hidden % 8 == 0");
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

int tile_weight_16x64(const int8_t* w, int8_t* tiled, int N, int K, hipStream_t s) {
  if (!w || !tiled || N <= 0 || K <= 0 || N % 16 != 0 || K % 64 != 0 || !aligned16(w) ||
      !aligned16(tiled))
    return lsh_fail(LSH_ERR_INVALID, "tile_weight_16x64: needs N % 16 == 0, K % 64 == 0, aligned pointers");
  const long chunks = (long)N * K / 16;
  tile_weight_16x64_kernel<<<(int)((chunks + 255) / 256), 256, 0, s>>>(w, tiled, N, K);
  return lsh_check_launch("tile_weight_16x64_kernel");
}

static thread_local hipEvent_t g_gln_ev_start = nullptr, g_gln_ev_stop = nullptr;
void gemm_ln_time_next_launch(hipEvent_t start, hipEvent_t stop) {
  g_gln_ev_start = start;
  g_gln_ev_stop = stop;
}

bool gemm_ln_fused_supported(int hidden, int K) {
  return hidden == K && (hidden == 512 || hidden == 768 || hidden == 1024);
}

template <typename T>
int gemm_i8_residual_ln_i8O(const int8_t* A, const int8_t* w_tiled, float alpha, const T* scale,
                            const T* bias, const T* residual_bias, int8_t* output, T* residual,
                            int batch_tokens, int hidden_size, int K, float dequant_scale,
                            float quant_scale, hipStream_t stream, bool is_post_ln) {
  if (!A || !w_tiled || !scale || !bias || !output || !residual || batch_tokens <= 0)
    return lsh_fail(LSH_ERR_INVALID, "gemm_i8_residual_ln_i8O: bad arguments");
  if (!gemm_ln_fused_supported(hidden_size, K))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "gemm_i8_residual_ln_i8O: needs hidden == K in {512, 768, 1024}");
  if (!aligned16(A) || !aligned16(w_tiled) || !aligned16(scale) || !aligned16(bias) ||
      !aligned16(residual_bias) || !aligned16(output) || !aligned16(residual))
    return lsh_fail(LSH_ERR_INVALID, "gemm_i8_residual_ln_i8O: pointers must be 16-byte aligned");
  const int grid = (batch_tokens + 15) / 16;
  // kernel-exact begin / end timestamps when the caller asked for them
  hipEvent_t e0 = g_gln_ev_start, e1 = g_gln_ev_stop;
  g_gln_ev_start = g_gln_ev_stop = nullptr;
  const int post = is_post_ln ? 1 : 0;
#define LSH_GLN(NT, KS, LPR, IT)                                                               \
  hipExtLaunchKernelGGL((gemm_ln_rows16_kernel<T, NT, KS, LPR, IT>), dim3(grid), dim3(512), 0,  \
                        stream, e0, e1, 0, A, w_tiled, alpha, residual, output, scale, bias,    \
                        residual_bias, batch_tokens, dequant_scale, quant_scale, post)
  if (hidden_size == 512) LSH_GLN(4, 8, 32, 2);
  else if (hidden_size == 768) LSH_GLN(6, 12, 32, 3);
  else LSH_GLN(8, 16, 64, 2);
#undef LSH_GLN
  return lsh_check_launch("gemm_ln_rows16_kernel");
}
template int gemm_i8_residual_ln_i8O<__half>(const int8_t*, const int8_t*, float, const __half*,
                                             const __half*, const __half*, int8_t*, __half*, int,
                                             int, int, float, float, hipStream_t, bool);
template int gemm_i8_residual_ln_i8O<float>(const int8_t*, const int8_t*, float, const float*,
                                            const float*, const float*, int8_t*, float*, int, int,
                                            int, float, float, hipStream_t, bool);

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
                         bool is_post_ln, const T* colsum, int nparts, long part_stride) {
  if (!input || !output || !scale || !bias || !residual)
    return lsh_fail(LSH_ERR_INVALID, "ker_residual_bias_ln_*_i8O: null pointer");
  return launch_ln<T, AccT, kLnResQuant>(input, residual, nullptr, output, scale, bias,
                                         residual_bias, colsum, batch_tokens, hidden_size,
                                         dequant_scale, quant_scale, is_post_ln, stream, nparts,
                                         part_stride);
}

template <typename T>
int residual_bias_ln_i32I(const int32_t* input, const T* scale, const T* bias, const T* residual,
                          T* output, int batch_tokens, int hidden_size, float dequant_scale,
                          hipStream_t stream, const T* colsum, int nparts, long part_stride) {
  if (!input || !output || !scale || !bias || !residual)
    return lsh_fail(LSH_ERR_INVALID, "ker_residual_bias_ln_i32I: null pointer");
  // the kernel only reads `residual`; output may alias it (the reference calls it in place)
  return launch_ln<T, int32_t, kLnResOut>(input, const_cast<T*>(residual), output, nullptr, scale,
                                          bias, nullptr, colsum, batch_tokens, hidden_size,
                                          dequant_scale, 0.f, 0, stream, nparts, part_stride);
}

#define LSH_INST(T)                                                                              \
  template int norm_layer_resual_i8O<T>(int, int, hipStream_t, T*, int8_t*, const T*, const T*,  \
                                        const T*, float, bool);                                  \
  template int residual_bias_ln_i8O<T, int8_t>(const int8_t*, const T*, const T*, const T*,      \
                                               int8_t*, T*, int, int, float, float, hipStream_t, \
                                               bool, const T*, int, long);                       \
  template int residual_bias_ln_i8O<T, int32_t>(const int32_t*, const T*, const T*, const T*,    \
                                                int8_t*, T*, int, int, float, float,             \
                                                hipStream_t, bool, const T*, int, long);         \
  template int residual_bias_ln_i32I<T>(const int32_t*, const T*, const T*, const T*, T*, int,   \
                                        int, float, hipStream_t, const T*, int, long);
LSH_INST(float)
LSH_INST(__half)
#undef LSH_INST

}  // namespace lsh
