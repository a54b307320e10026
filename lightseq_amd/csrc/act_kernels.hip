// dequant + bias + GELU/ReLU + requant, int8 -> int8, one HBM pass (2 B/element).
//
// 16 consecutive codes per thread (one 16-byte load, one 16-byte store).
// Replaces inference/kernels/transformerKernels_int8.cc.cu:865-1078.
//
// The output code is a function of the input code and the column alone, and the GELU costs
// ~30 vector instructions per element: with a few thousand rows it is cheaper to tabulate
// the 256 codes of each column once per workgroup in LDS and to look every element up
// (bias_act_lut_kernel) than to evaluate the function per element -- the table entries come
// from the same routine, so the bytes are the same.
#include "ls_device.h"
#include "ls_launch.h"

#include <atomic>

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

// One workgroup tabulates kLutCols columns (a 32- or 64-byte slice of each row) and applies
// the table to `rows_per_chunk` rows.  Neighbouring slices share a 128-byte line of memory:
// when the slice count allows, the workgroups of four neighbouring slices run on the same XCD
// (workgroup w runs on XCD w % 8) one after the other, so the line leaves HBM once.

template <typename T, int ACT, int kLutCols>
__global__ void __launch_bounds__(512)
bias_act_lut_kernel(const int8_t* in, int8_t* out, const T* __restrict__ bias, int tokens,
                    int feat, int rows_per_chunk, int nchunks, float ds, float qs,
                    float clip_max) {
  constexpr int kLutTpr = kLutCols / 16;   // threads per row
  constexpr int kLutRows = 512 / kLutTpr;  // rows per pass of the workgroup
  __shared__ __align__(16) uint8_t lut[kLutCols * 256];
  const int nstrips = feat / kLutCols;
  int strip, chunk;
  if ((nstrips & 3) == 0) {
    const int xcd = blockIdx.x & 7, k = blockIdx.x >> 3;
    const int task = (k >> 2) * 8 + xcd;  // a line's four slices over one chunk of rows
    const int groups = nstrips >> 2;
    if (task >= groups * nchunks) return;
    strip = (task % groups) * 4 + (k & 3);
    chunk = task / groups;
  } else {
    strip = blockIdx.x % nstrips;
    chunk = blockIdx.x / nstrips;
    if (chunk >= nchunks) return;
  }
  const int col0 = strip * kLutCols;
  // thread: 16 consecutive columns of one row in kLutRows
  const int half = threadIdx.x % kLutTpr;
  const int row_end = min((chunk + 1) * rows_per_chunk, tokens);
  const long off = (long)col0 + half * 16;
  constexpr int UNR = 4, STEP = kLutRows * UNR;  // rows in flight per thread and buffer
  uint4 wa[UNR], wb[UNR];
  auto fetch = [&](uint4 (&w)[UNR], int row) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int r = row + kLutRows * u;
      if (r < row_end) w[u] = *reinterpret_cast<const uint4*>(in + (long)r * feat + off);
    }
  };
  const uint8_t* tab = lut + half * 16 * 256;
  auto apply = [&](const uint4 (&w)[UNR], int row) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int r = row + kLutRows * u;
      if (r >= row_end) break;
      const uint32_t wi[4] = {w[u].x ^ 0x80808080u, w[u].y ^ 0x80808080u, w[u].z ^ 0x80808080u,
                              w[u].w ^ 0x80808080u};  // code + 128 in every byte
      uint32_t wo[4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint32_t o = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k)
          o |= (uint32_t)tab[(g * 4 + k) * 256 + ((wi[g] >> (8 * k)) & 0xff)] << (8 * k);
        wo[g] = o;
      }
      *reinterpret_cast<uint4*>(out + (long)r * feat + off) = make_uint4(wo[0], wo[1], wo[2], wo[3]);
    }
  };
  // the first rows travel while the table is computed
  int row = chunk * rows_per_chunk + threadIdx.x / kLutTpr;
  fetch(wa, row);
  fetch(wb, row + STEP);
  for (int e = threadIdx.x; e < kLutCols * 256; e += 512) {
    const int c = e >> 8, code = (e & 255) - 128;
    lut[e] = (uint8_t)dequant_bias_act_requant<ACT>(code, ds, TT<T>::ld(bias, col0 + c), qs,
                                                    clip_max);
  }
  __syncthreads();
  for (; row < row_end; row += 2 * STEP) {
    apply(wa, row);
    fetch(wa, row + 2 * STEP);
    apply(wb, row + STEP);
    fetch(wb, row + 3 * STEP);
  }
}

static std::atomic<bool> g_act_lut_enabled{true};
bool bias_act_enable_lut_kernel(bool on) {
  const bool prev = g_act_lut_enabled.exchange(on);
  if (prev != on) route_epoch_bump();
  return prev;
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
  // The table pays once a workgroup has ~2000 rows to apply it to and the function is dear.
  // Slices of 32 columns keep the table small (what counts with few rows); with many rows
  // 64-byte slices, whole sectors of memory, stream faster.
  if (vec && ACT == kActGelu && feat % 64 == 0 && tokens >= 1024 &&
      g_act_lut_enabled.load(std::memory_order_relaxed)) {
    const int cols = tokens >= 16384 ? 64 : 32;
    const int nstrips = feat / cols;
    int nchunks = (tokens + 2047) / 2048;
    // few columns: more, shorter chunks keep the compute units busy (not below 512 rows)
    while (nstrips * nchunks < 192 && tokens / (nchunks * 2) >= 512) nchunks *= 2;
    const int rows_per_chunk = (tokens + nchunks - 1) / nchunks;
    int grid = nstrips * nchunks;
    if ((nstrips & 3) == 0) grid = ((nstrips / 4 * nchunks + 7) / 8) * 32;
    if (cols == 64)
      bias_act_lut_kernel<T, ACT, 64><<<grid, 512, 0, s>>>(input, output, bias, tokens, feat,
                                                           rows_per_chunk, nchunks, ds, qs,
                                                           clip_max);
    else
      bias_act_lut_kernel<T, ACT, 32><<<grid, 512, 0, s>>>(input, output, bias, tokens, feat,
                                                           rows_per_chunk, nchunks, ds, qs,
                                                           clip_max);
    return lsh_check_launch("bias_act_lut_kernel");
  }
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
