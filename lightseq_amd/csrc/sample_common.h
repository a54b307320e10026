// Device-side pieces shared by the random-sampling kernels of the GPT model (gpt_kernels.hip)
// and of the encoder-decoder model (sample_kernels.hip): the generator state and its uniform
// numbers, the workgroup's shared block, and the choice of a token from one candidate per
// thread.  Both kernel families restate the reference with the 1024 threads per block its
// models launch them with (inference/kernels/gptKernels_int8.cc.cu:252-640,
// transformerKernels_int8.cc.cu:1908-2290).
#pragma once

#include "ls_device.h"

namespace lsh {

struct alignas(16) SampleState {
  unsigned long long seed;
  unsigned int row, draws;
};
static_assert(sizeof(SampleState) == 16, "lsh_rng_state_t is 16 bytes");

__device__ __forceinline__ uint32_t philox4x32_10_word0(uint32_t c0, uint32_t c1, uint32_t c2,
                                                        uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const unsigned long long p0 = 0xD2511F53ull * c0, p1 = 0xCD9E8D57ull * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

constexpr int kSampleThreads = 1024;
constexpr int kSampleIdBits = 20, kSampleIdMask = (1 << kSampleIdBits) - 1;

struct SampleShared {
  int cls[kSampleThreads];   // class maxima (codes; -129 = empty), then candidate keys
  float pf[kSampleThreads];  // exps (top-p), then wavefront prefix totals
  int hist[260];             // classes per maximum code (top-p)
  float red[16];
  int thr, tok;
  float x;
};

// The next uniform number in (0, 1] of one sequence (called by one thread): word 0 of
// Philox4x32-10 with key = seed and counter = (draws, 0, row, 0), mapped as curand_uniform maps
// 32 bits; advances the state.
__device__ __forceinline__ float sample_draw_uniform(SampleState* st) {
  const SampleState s = *st;
  const uint32_t w = philox4x32_10_word0(s.draws, 0u, s.row, 0u, (uint32_t)s.seed,
                                         (uint32_t)(s.seed >> 32));
  st->draws = s.draws + 1;
  return (float)w * 2.3283064365386963e-10f + 1.1641532182693481e-10f;
}

// Thread t holds at most one candidate: its exp `ex` (0 = none) and id `my_id`; sh.x holds the
// uniform number.  Probabilities, inclusive prefix in thread order, the first thread whose
// prefix reaches x (gptKernels_int8.cc.cu:347-395); every thread returns the chosen id.
__device__ __forceinline__ int sample_pick(float ex, int my_id, SampleShared& sh) {
  const int t = threadIdx.x;
  const float prob = ex / block_sum(ex, sh.red);
  // inclusive prefix in thread order: within the wavefront, then the totals of the wavefronts before
  float pre = prob;
  const int lane = t & 63, wid = t >> 6;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const float up = __shfl_up(pre, d);
    if (lane >= d) pre += up;
  }
  __syncthreads();
  if (lane == 63) sh.pf[wid] = pre;
  __syncthreads();
  for (int w = 0; w < wid; ++w) pre += sh.pf[w];
  const float x = sh.x;
  int pick = kSampleThreads - (int)block_max((float)(x > pre ? 0 : kSampleThreads - t), sh.red);
  if (pick == kSampleThreads) {
    // rounding left the last prefix below x: the lowest thread of the largest probability
    const float pmax = block_max(prob, sh.red);
    pick = kSampleThreads - (int)block_max((float)(prob == pmax ? kSampleThreads - t : 0), sh.red);
  }
  if (t == pick) sh.tok = my_id;
  __syncthreads();
  return sh.tok;
}

}  // namespace lsh
