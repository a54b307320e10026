// Per-tensor symmetric quantise / dequantise, weight quantise+transpose and the
// scaled column sum used by the ReLU offset trick.  All streaming, HBM-bound.
//
// Replaces inference/kernels/transformerKernels_int8.cc.cu:29-147,
// inference/model/cublas_helper.cc:502-605 (quantize_weight + layout transform)
// and inference/kernels/transformerKernels.cc.cu:18-80.
#include "ls_device.h"
#include "ls_launch.h"

namespace lsh {

// 8 elements per thread: 16 B (fp16) or 2x16 B (fp32) in, 8 B out.
template <typename T>
__global__ void __launch_bounds__(256)
quantize8_kernel(const T* __restrict__ in, int8_t* __restrict__ out, long n8, float qs) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < n8; i += stride) {
    float a[4], b[4];
    ld4(in, i * 8, a);
    ld4(in, i * 8 + 4, b);
    uint2 o;
    o.x = pack4_i8(float2int8(a[0], qs), float2int8(a[1], qs), float2int8(a[2], qs),
                   float2int8(a[3], qs));
    o.y = pack4_i8(float2int8(b[0], qs), float2int8(b[1], qs), float2int8(b[2], qs),
                   float2int8(b[3], qs));
    *reinterpret_cast<uint2*>(out + i * 8) = o;
  }
}

template <typename T>
__global__ void quantize1_kernel(const T* __restrict__ in, int8_t* __restrict__ out, long start,
                                 long n, float qs) {
  long i = start + (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (int8_t)float2int8(TT<T>::ld(in, i), qs);
}

template <typename T>
__global__ void __launch_bounds__(256)
dequantize4_kernel(const int32_t* __restrict__ in, T* __restrict__ out, long n4, float ds) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < n4; i += stride) {
    int4 w = *reinterpret_cast<const int4*>(in + i * 4);
    float o[4] = {(float)w.x * ds, (float)w.y * ds, (float)w.z * ds, (float)w.w * ds};
    st4(out, i * 4, o);
  }
}

template <typename T>
__global__ void dequantize1_kernel(const int32_t* __restrict__ in, T* __restrict__ out,
                                   long start, long n, float ds) {
  long i = start + (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) TT<T>::st(out, i, (float)in[i] * ds);
}

static int stream_grid(long work_items, int block) {
  long g = (work_items + block - 1) / block;
  const long cap = 256L * 16;  // 16 resident workgroups per CU is plenty to saturate HBM
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename T>
int quantize_tensor(const T* input, int8_t* output, long n, float quant_scale, hipStream_t s) {
  if (n < 0 || (n > 0 && (!input || !output)))
    return lsh_fail(LSH_ERR_INVALID, "launch_quantize_tensor: bad arguments");
  if (n == 0) return LSH_OK;
  long n8 = (aligned16(input) && aligned16(output)) ? n / 8 : 0;
  if (n8 > 0)
    quantize8_kernel<T><<<stream_grid(n8, 256), 256, 0, s>>>(input, output, n8, quant_scale);
  long rest = n - n8 * 8;
  if (rest > 0)
    quantize1_kernel<T><<<(int)((rest + 255) / 256), 256, 0, s>>>(input, output, n8 * 8, n,
                                                                   quant_scale);
  return lsh_check_launch("quantize_tensor");
}

template <typename T>
int dequantize_tensor(const int32_t* input, T* output, long n, float dequant_scale,
                      hipStream_t s) {
  if (n < 0 || (n > 0 && (!input || !output)))
    return lsh_fail(LSH_ERR_INVALID, "launch_dequantize_tensor: bad arguments");
  if (n == 0) return LSH_OK;
  long n4 = (aligned16(input) && aligned16(output)) ? n / 4 : 0;
  if (n4 > 0)
    dequantize4_kernel<T><<<stream_grid(n4, 256), 256, 0, s>>>(input, output, n4, dequant_scale);
  long rest = n - n4 * 4;
  if (rest > 0)
    dequantize1_kernel<T><<<(int)((rest + 255) / 256), 256, 0, s>>>(input, output, n4 * 4, n,
                                                                     dequant_scale);
  return lsh_check_launch("dequantize_tensor");
}

// in: rows x cols -> out: cols x rows int8 (or rows x cols when !TRANSPOSE).
// 64x64 tiles through LDS so both sides are coalesced.
template <typename T, bool TRANSPOSE>
__global__ void __launch_bounds__(256)
quantize_transpose_kernel(const T* __restrict__ in, int8_t* __restrict__ out, int rows, int cols,
                          float qs) {
  __shared__ int8_t tile[64][65];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    int rr = r0 + r, cc = c0 + tx;
    if (rr < rows && cc < cols) tile[r][tx] = (int8_t)float2int8(TT<T>::ld(in, (long)rr * cols + cc), qs);
  }
  __syncthreads();
  if (TRANSPOSE) {
    for (int c = ty; c < 64; c += 4) {
      int cc = c0 + c, rr = r0 + tx;
      if (rr < rows && cc < cols) out[(long)cc * rows + rr] = tile[tx][c];
    }
  } else {
    for (int r = ty; r < 64; r += 4) {
      int rr = r0 + r, cc = c0 + tx;
      if (rr < rows && cc < cols) out[(long)rr * cols + cc] = tile[r][tx];
    }
  }
}

template <typename T>
int quantize_transpose(const T* input, int8_t* output, int rows, int cols, float quant_scale,
                       bool transpose, hipStream_t s) {
  if (rows <= 0 || cols <= 0 || !input || !output)
    return lsh_fail(LSH_ERR_INVALID, "quantize_weight: bad arguments");
  dim3 grid((cols + 63) / 64, (rows + 63) / 64);
  if (transpose)
    quantize_transpose_kernel<T, true><<<grid, 256, 0, s>>>(input, output, rows, cols, quant_scale);
  else
    quantize_transpose_kernel<T, false><<<grid, 256, 0, s>>>(input, output, rows, cols, quant_scale);
  return lsh_check_launch("quantize_transpose_kernel");
}

// out[c] = T(scale * sum_r inp[r, c]).  64 columns x 4 row-slices per workgroup.
template <typename T>
__global__ void __launch_bounds__(256)
scaled_colsum_kernel(const T* __restrict__ inp, T* __restrict__ out, int rows, int cols,
                     float scale) {
  __shared__ float part[4][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + tx;
  float s = 0.f;
  if (c < cols)
    for (int r = ty; r < rows; r += 4) s += TT<T>::ld(inp, (long)r * cols + c);
  part[ty][tx] = s;
  __syncthreads();
  if (ty == 0 && c < cols)
    TT<T>::st(out, c, (part[0][tx] + part[1][tx] + part[2][tx] + part[3][tx]) * scale);
}

template <typename T>
int scaled_colsum(const T* inp, T* out, int rows, int cols, float scale, hipStream_t s) {
  if (rows <= 0 || cols <= 0 || !inp || !out)
    return lsh_fail(LSH_ERR_INVALID, "launch_scaled_colsum: bad arguments");
  scaled_colsum_kernel<T><<<(cols + 63) / 64, 256, 0, s>>>(inp, out, rows, cols, scale);
  return lsh_check_launch("scaled_colsum_kernel");
}

// Stored model kernels are uint8 = code + 127 (training/ops/pytorch/export_quant.py:12-20).
// rows x cols bytes -> int8 codes clamped to [-127, 127], optionally transposed.
template <bool TRANSPOSE>
__global__ void __launch_bounds__(256)
stored_u8_to_i8_kernel(const uint8_t* __restrict__ in, int8_t* __restrict__ out, int rows,
                       int cols) {
  __shared__ int8_t tile[64][65];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    int rr = r0 + r, cc = c0 + tx;
    if (rr < rows && cc < cols) {
      int q = (int)in[(long)rr * cols + cc] - 127;
      tile[r][tx] = (int8_t)max(-127, min(127, q));
    }
  }
  __syncthreads();
  if (TRANSPOSE) {
    for (int c = ty; c < 64; c += 4) {
      int cc = c0 + c, rr = r0 + tx;
      if (rr < rows && cc < cols) out[(long)cc * rows + rr] = tile[tx][c];
    }
  } else {
    for (int r = ty; r < 64; r += 4) {
      int rr = r0 + r, cc = c0 + tx;
      if (rr < rows && cc < cols) out[(long)rr * cols + cc] = tile[r][tx];
    }
  }
}

int stored_u8_to_i8(const uint8_t* input, int8_t* output, int rows, int cols, bool transpose,
                    hipStream_t s) {
  if (rows <= 0 || cols <= 0 || !input || !output)
    return lsh_fail(LSH_ERR_INVALID, "stored_u8_to_i8: bad arguments");
  dim3 grid((cols + 63) / 64, (rows + 63) / 64);
  if (transpose)
    stored_u8_to_i8_kernel<true><<<grid, 256, 0, s>>>(input, output, rows, cols);
  else
    stored_u8_to_i8_kernel<false><<<grid, 256, 0, s>>>(input, output, rows, cols);
  return lsh_check_launch("stored_u8_to_i8_kernel");
}

// T((uint8 - 127) * clip_max / 127): the loader's dequantize() followed by its cast
// to T (inference/tools/util.cc.cu:346-348, proto/quant_bert_weight.cc:28-30).
template <typename T>
__global__ void stored_u8_dequant_kernel(const uint8_t* __restrict__ in, T* __restrict__ out,
                                         long n, float clip_max) {
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long stride = (long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) TT<T>::st(out, i, ((float)in[i] - 127.f) * clip_max / 127.f);
}

template <typename T>
int stored_u8_dequant(const uint8_t* input, T* output, long n, float clip_max, hipStream_t s) {
  if (n <= 0 || !input || !output)
    return lsh_fail(LSH_ERR_INVALID, "stored_u8_dequant: bad arguments");
  stored_u8_dequant_kernel<T><<<stream_grid(n, 256), 256, 0, s>>>(input, output, n, clip_max);
  return lsh_check_launch("stored_u8_dequant_kernel");
}
template int stored_u8_dequant<float>(const uint8_t*, float*, long, float, hipStream_t);
template int stored_u8_dequant<__half>(const uint8_t*, __half*, long, float, hipStream_t);

// A fill kernel for the words a generation step must clear: a memset node in a captured
// graph replays wrongly on this platform, a kernel node does not.
__global__ void fill_i32_kernel(int* __restrict__ p, int value, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}
int fill_i32(int* p, int value, int n, hipStream_t s) {
  if (!p || n <= 0) return lsh_fail(LSH_ERR_INVALID, "fill_i32: bad arguments");
  fill_i32_kernel<<<(n + 255) / 256, 256, 0, s>>>(p, value, n);
  return lsh_check_launch("fill_i32_kernel");
}

#define LSH_INST(T)                                                                          \
  template int quantize_tensor<T>(const T*, int8_t*, long, float, hipStream_t);              \
  template int dequantize_tensor<T>(const int32_t*, T*, long, float, hipStream_t);           \
  template int quantize_transpose<T>(const T*, int8_t*, int, int, float, bool, hipStream_t); \
  template int scaled_colsum<T>(const T*, T*, int, int, float, hipStream_t);
LSH_INST(float)
LSH_INST(__half)
#undef LSH_INST

}  // namespace lsh
