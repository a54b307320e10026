// fp16 GEMM with fp32 accumulation on v_mfma_f32_32x32x16_f16:
//   C[M,N] = A[M,K] * W[N,K]^T, both operands K-contiguous, C row-major.
//
// Used once per translation request to project the encoder output onto the keys and
// values of every decoder layer (inference/model/quant_decoder.cc.cu:489-501), so it
// is written for simplicity: a workgroup of 4 wavefronts owns a 64 x 128 tile, each
// wavefront a 64 x 32 slice of it, and the MFMA operands are loaded straight from
// global memory (one 16-byte row fragment per lane and k-step; rows beyond the
// matrix are clamped for the loads and masked for the stores).
#include "ls_device.h"
#include "ls_launch.h"

namespace lsh {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(256)
gemm_f16_nt_kernel(const __half* __restrict__ A, const __half* __restrict__ W,
                   __half* __restrict__ C, int M, int N, int K) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int row0 = blockIdx.y * 64;
  const int col0 = blockIdx.x * 128 + wid * 32;
  if (col0 >= N) return;  // whole wavefront outside the matrix; no barriers are used
  const int r = lane & 31, kc = (lane >> 5) * 8;
  // operand rows of this lane, clamped into the matrices
  const long a0 = (long)min(row0 + r, M - 1) * K + kc;
  const long a1 = (long)min(row0 + 32 + r, M - 1) * K + kc;
  const long b0 = (long)min(col0 + r, N - 1) * K + kc;
  f32x16 acc0 = {0}, acc1 = {0};
  for (int k = 0; k < K; k += 16) {
    const f16x8 av0 = *reinterpret_cast<const f16x8*>(A + a0 + k);
    const f16x8 av1 = *reinterpret_cast<const f16x8*>(A + a1 + k);
    const f16x8 bv = *reinterpret_cast<const f16x8*>(W + b0 + k);
    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(av0, bv, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(av1, bv, acc1, 0, 0, 0);
  }
  // acc[v] holds row 8*(v/4) + 4*(lane/32) + v%4, column lane%32 of the 32x32 tile
  const int col = col0 + r;
  if (col < N) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int rr = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      if (row0 + rr < M) C[(long)(row0 + rr) * N + col] = __float2half_rn(acc0[v]);
      if (row0 + 32 + rr < M) C[(long)(row0 + 32 + rr) * N + col] = __float2half_rn(acc1[v]);
    }
  }
}

int gemm_f16_nt(const __half* A, const __half* W, __half* C, int M, int N, int K, hipStream_t s) {
  if (!A || !W || !C || M <= 0 || N <= 0 || K <= 0)
    return lsh_fail(LSH_ERR_INVALID, "fp16 gemm: bad arguments");
  if (K % 16 != 0) return lsh_fail(LSH_ERR_UNSUPPORTED, "fp16 gemm: K must be a multiple of 16");
  if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W)) & 15u)
    return lsh_fail(LSH_ERR_INVALID, "fp16 gemm: operands must be 16-byte aligned");
  dim3 grid((N + 127) / 128, (M + 63) / 64);
  if (grid.y > 65535) return lsh_fail(LSH_ERR_UNSUPPORTED, "fp16 gemm: M too large");
  gemm_f16_nt_kernel<<<grid, 256, 0, s>>>(A, W, C, M, N, K);
  return lsh_check_launch("gemm_f16_nt_kernel");
}

// StridedBatchGemm<T>::Forward (ops/includes/strided_batch_gemm.h:45-57,
// cublas_strided_batched_gemm of kernels/cuda/cublas_wrappers.cpp): per batch, in cuBLAS's
// column-major terms, C (m x n) = alpha * op(A) (m x k) * op(B) (k x n) + beta * C with
// strides m*k, n*k, m*n.  Read as row-major arrays: out[n][m]; A is [m][k] when op_A = T and
// [k][m] when N; B is [n][k] when op_B = N and [k][n] when T.  fp32 accumulation, one thread
// per output element (m fastest): the layers of this library run the fused attention kernel,
// this stand-alone form exists for callers of the operator and is written for clarity.
template <typename T>
__global__ void __launch_bounds__(256)
strided_batch_gemm_kernel(const T* __restrict__ A, const T* __restrict__ B, T* C, int m, int n,
                          int k, float alpha, float beta, int ta, int tb, long total) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int i = (int)(idx % m);
  const long r = idx / m;
  const int j = (int)(r % n);
  const long b = r / n;
  const T* a = A + b * (long)m * k;
  const T* bb = B + b * (long)n * k;
  const long a_step = ta ? 1 : m, a0 = ta ? (long)i * k : i;
  const long b_step = tb ? n : 1, b0 = tb ? j : (long)j * k;
  float acc = 0.f;
  for (int kk = 0; kk < k; ++kk)
    acc = fmaf((float)a[a0 + kk * a_step], (float)bb[b0 + kk * b_step], acc);
  float v = alpha * acc;
  if (beta != 0.f) v += beta * (float)C[idx];
  C[idx] = (T)v;
}

template <typename T>
int strided_batch_gemm(int bsz, int m, int n, int k, float alpha, float beta, int op_a, int op_b,
                       const T* A, const T* B, T* C, hipStream_t s) {
  if (!A || !B || !C || bsz <= 0 || m <= 0 || n <= 0 || k <= 0)
    return lsh_fail(LSH_ERR_INVALID, "StridedBatchGemm: bad arguments");
  if ((op_a != 0 && op_a != 1) || (op_b != 0 && op_b != 1))
    return lsh_fail(LSH_ERR_INVALID, "StridedBatchGemm: op must be 0 (N) or 1 (T)");
  const long total = (long)bsz * m * n;
  if ((total + 255) / 256 > 0x7fffffffL)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "StridedBatchGemm: too many output elements");
  strided_batch_gemm_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, s>>>(
      A, B, C, m, n, k, alpha, beta, op_a, op_b, total);
  return lsh_check_launch("strided_batch_gemm_kernel");
}
template int strided_batch_gemm<__half>(int, int, int, int, float, float, int, int, const __half*,
                                        const __half*, __half*, hipStream_t);
template int strided_batch_gemm<float>(int, int, int, int, float, float, int, int, const float*,
                                       const float*, float*, hipStream_t);

}  // namespace lsh
