// fp16 GEMM with fp32 accumulation on v_mfma_f32_32x32x16_f16:
//   C[M,N] = A[M,K] * W[N,K]^T, both operands K-contiguous, C row-major.
//
// Used once per translation request to project the encoder output onto the keys and
// values of every decoder layer (inference/model/quant_decoder.cc.cu:489-501), so it
// is written for simplicity: a workgroup of 4 wavefronts owns a 64 x 128 tile, each
// wavefront a 64 x 32 slice of it, and the MFMA operands are loaded straight from
// global memory (one 16-byte row fragment per lane and k-step; rows beyond the
// matrix are clamped for the loads and masked for the stores).
#include "ls_device.cuh"
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

}  // namespace lsh
