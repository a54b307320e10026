// int8 x int8 -> int32 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8),
// with requantising and fused epilogues.
//
//   C[M,N] = epilogue( sum_k A[M,k] * W[N,k] )        A, W: K-contiguous int8
//
// Replaces the cuBLASLt int8 GEMMs and their tuned-algorithm table
// (inference/model/cublas_helper.cc:31-225,361-489, cublas_algo_map.cc).
//
// Four kernels share the epilogues:
//
//  * gemm_i8_skinny_kernel -- M <= 64 (decode steps), K % 128 == 0.  A workgroup owns 32
//    output columns for all rows; its 4 wavefronts split the 128-byte K chunks of the
//    workgroup's K range, load operands from global memory straight into MFMA registers
//    (no LDS staging, no barrier in the loop) and sum their partial tiles through LDS.
//    The weight matrix is read once, by ceil(N/32) * ksplit workgroups; with ksplit > 1
//    range p stores its int32 partial sums to plane p of the output ([ksplit][M][N]).
//  * gemm_i8_stream_kernel -- the fast path (K % 128 == 0).  Persistent: 2 workgroups
//    per compute unit walk a list of 128x64 tiles; operand stages (128 rows of A and 64 of
//    W, 128 B each) are brought from L2 straight into LDS with global_load_lds_dwordx4
//    (no VGPR staging) into a 3-stage ring, and the prefetch cursor runs two K steps ahead
//    of the compute cursor across tile boundaries, so a tile's first loads are in flight
//    while the previous tile is still in its K loop / epilogue.  K loops of fewer than 12
//    steps use a 2-stage ring and 3 workgroups per compute unit; the tabulated epilogue
//    keeps the table rows of its tile in LDS behind a 2-stage ring.
//  * gemm_i8_stream128_kernel -- the same path with 128x128 tiles and a 2-stage ring, for
//    the epilogues that read global memory and for short K loops over many tiles.
//  * gemm_i8_generic_kernel -- any K % 16 == 0, any alignment of M and N: register
//    staged, zero-filled tails, one tile per workgroup.
//
// Common geometry.  256 threads = 4 wavefronts (2x2); per wavefront 64x64 accumulators as
// 2x2 MFMA blocks (64x32 as 2x1 in the fast path).  LDS rows are 128 B = eight 16-byte chunks, XOR swizzled for the
// 64-bank LDS (a ds_read_b128 is served 16 lanes per clock; the 16 lanes must hit 16
// distinct 16-byte slots of a 256-byte window).  The W tile is the MFMA "A" operand so
// that consecutive accumulator registers of a lane run along N, and the W rows fed to
// the MFMA are permuted (sigma) so that the 16 accumulators of a lane are 16 adjacent
// columns of C: one 16-byte store for int8 output, two for fp16.
#include "ls_device.h"
#include "ls_launch.h"
#include "tile_common.h"
#include "gemm_tile.h"

#include <hip/hip_ext.h>

#include <atomic>
#include <cstdlib>
#include <mutex>
#include <string>
#include <type_traits>

namespace lsh {

constexpr int kBM = 128, kBN = 128;

// n / d for 0 <= n < 2^24, d > 0, with inv = 1.0f / d from the host: the float product is
// within one of the quotient, the remainder decides.  A handful of instructions where the
// integer division is about forty -- in kernels whose length is their instruction count.
__device__ __forceinline__ int div_by(int n, int d, float inv) {
  int q = (int)((float)n * inv);
  const int r = n - q * d;
  if (r >= d) ++q;
  if (r < 0) --q;
  return q;
}

// Decode-step QKV product followed by ker_arrange_decself_qkv_i8I_i8O
// (inference/kernels/transformerKernels_int8.cc.cu:1432-1513; call sites
// model/quant_decoder.cc.cu:660-674, model/quant_gpt_encoder.cc.cu:640-653): the int8 code
// of the product is dequantised, biased and requantised with the cache scale; columns
// [0, H) go to new_q [M, H], [H, 2H) and [2H, 3H) to slot step_id of the K and V caches
// [M, heads, max_step, d].  Same float arithmetic as the stand-alone kernel (no fused
// multiply-add).
struct EpiDecQkvI8 {
  int8_t *new_q, *new_k, *new_v;
  const __half* bias;
  float alpha, dequant_scale, quant_scale;
  int hidden, head_num, dim_per_head, max_step, step_id;
  float inv_hidden, inv_dim;  // 1 / hidden, 1 / dim_per_head (for store1)
  // the 16 bias values of columns n .. n + 15: they do not depend on the product, so the
  // decode-step kernel requests them with its first weights
  struct Pre {
    half8_t b0, b1;
  };
  __device__ __forceinline__ Pre prefetch(int n) const {
    return Pre{*reinterpret_cast<const half8_t*>(bias + n),
               *reinterpret_cast<const half8_t*>(bias + n + 8)};
  }
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    store16_pre(m, n, N, c, full, prefetch(n));
  }
  __device__ __forceinline__ void store16_pre(long m, int n, int N, const v16i& c, bool,
                                              const Pre& pre) const {
#pragma clang fp contract(off)
    const int part = n / hidden, i = n - part * hidden;
    const half8_t b0 = pre.b0, b1 = pre.b1;
    int q[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float b = __half2float(k < 8 ? b0.v[k] : b1.v[k - 8]);
      const float val = (float)requant_acc(c[k], alpha) * dequant_scale + b;
      q[k] = float2int8(val, quant_scale);
    }
    int8_t* dst;
    if (part == 0) {
      dst = new_q + m * hidden + i;
    } else {
      const int head = i / dim_per_head, dim = i - head * dim_per_head;
      dst = (part == 1 ? new_k : new_v) +
            ((m * head_num + head) * max_step + step_id) * dim_per_head + dim;
    }
    uint4 o;
    o.x = pack4_i8(q[0], q[1], q[2], q[3]);
    o.y = pack4_i8(q[4], q[5], q[6], q[7]);
    o.z = pack4_i8(q[8], q[9], q[10], q[11]);
    o.w = pack4_i8(q[12], q[13], q[14], q[15]);
    *reinterpret_cast<uint4*>(dst) = o;
    (void)N;
  }
  // one element; its bias value is requested with the first weights
  struct Pre1 {
    __half b;
  };
  __device__ __forceinline__ Pre1 prefetch1(int n) const { return Pre1{bias[n]}; }
  // what the elements of one column share: the 16 columns of a block lie in one part and one
  // head (dim_per_head % 16 == 0), so the divisions run on the block's first column, the same
  // in every lane, once per block; an element's address is base + row * row_stride + add.
  // 32-bit offsets: this form serves the decode-step kernels only (at most 64 rows; the
  // launcher refuses caches of 2^31 bytes and more for them)
  struct Blk1 {
    int8_t* base;
    int row_stride, add;
  };
  __device__ __forceinline__ Blk1 block1(int n) const {
    const int nb = __builtin_amdgcn_readfirstlane(n & ~15);
    const int part = div_by(nb, hidden, inv_hidden), ib = nb - part * hidden;
    const int head = div_by(ib, dim_per_head, inv_dim), dim = ib - head * dim_per_head + (n & 15);
    if (part == 0) return Blk1{new_q, hidden, ib + (n & 15)};
    return Blk1{part == 1 ? new_k : new_v, head_num * max_step * dim_per_head,
                (head * max_step + step_id) * dim_per_head + dim};
  }
  __device__ __forceinline__ void store1(long m, Blk1 blk, int N, int acc, Pre1 pre,
                                         const int8_t*, int) const {
#pragma clang fp contract(off)
    const float val = (float)requant_acc_fast(acc, alpha) * dequant_scale + __half2float(pre.b);
    blk.base[(unsigned)((int)m * blk.row_stride + blk.add)] =
        (int8_t)float2int8(val, quant_scale);
    (void)N;
  }
  bool vec_ok(int) const { return true; }
  static const char* name() { return "EpiDecQkvI8"; }
};

// Decode-step cross-attention query product followed by ker_arrange_encdec_q_i8I
// (inference/kernels/transformerKernels_int8.cc.cu:1596-1645; call site
// model/quant_decoder.cc.cu:745-760): code -> half(code * dq) + bias (a half add) -> fp16 q
// [batch, heads, beam, d].
struct EpiEncdecQF16 {
  __half* new_q;
  const __half* bias;
  float alpha, dequant_scale;
  int beam_size, head_num, dim_per_head;
  float inv_beam, inv_dim;  // 1 / beam_size, 1 / dim_per_head (for store1)
  struct Pre {  // the bias of columns n .. n + 15, requested ahead of the product
    half8_t b0, b1;
  };
  __device__ __forceinline__ Pre prefetch(int n) const {
    return Pre{*reinterpret_cast<const half8_t*>(bias + n),
               *reinterpret_cast<const half8_t*>(bias + n + 8)};
  }
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    store16_pre(m, n, N, c, full, prefetch(n));
  }
  __device__ __forceinline__ void store16_pre(long m, int n, int N, const v16i& c, bool,
                                              const Pre& pre) const {
    const int head = n / dim_per_head, dim = n - head * dim_per_head;
    const long batch_id = m / beam_size, beam_id = m - batch_id * beam_size;
    __half* dst = new_q + ((batch_id * head_num + head) * beam_size + beam_id) * dim_per_head + dim;
    const half8_t b0 = pre.b0, b1 = pre.b1;
    half8_t lo, hi;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      lo.v[k] = __float2half_rn(dequant_add_bias_h(requant_acc(c[k], alpha), dequant_scale,
                                                   __half2float(b0.v[k])));
      hi.v[k] = __float2half_rn(dequant_add_bias_h(requant_acc(c[8 + k], alpha), dequant_scale,
                                                   __half2float(b1.v[k])));
    }
    *reinterpret_cast<half8_t*>(dst) = lo;
    *reinterpret_cast<half8_t*>(dst + 8) = hi;
    (void)N;
  }
  struct Pre1 {
    __half b;
  };
  __device__ __forceinline__ Pre1 prefetch1(int n) const { return Pre1{bias[n]}; }
  struct Blk1 {
    int add;  // the column's share of the offset: head * beam_size * dim_per_head + dim
  };
  __device__ __forceinline__ Blk1 block1(int n) const {
    const int nb = __builtin_amdgcn_readfirstlane(n & ~15);
    const int head = div_by(nb, dim_per_head, inv_dim), dim = nb - head * dim_per_head + (n & 15);
    return Blk1{head * beam_size * dim_per_head + dim};
  }
  __device__ __forceinline__ void store1(long m, Blk1 blk, int N, int acc, Pre1 pre,
                                         const int8_t*, int) const {
    const int batch_id = div_by((int)m, beam_size, inv_beam), beam_id = (int)m - batch_id * beam_size;
    new_q[(unsigned)((batch_id * head_num * beam_size + beam_id) * dim_per_head + blk.add)] =
        __float2half_rn(dequant_add_bias_h(requant_acc_fast(acc, alpha), dequant_scale,
                                           __half2float(pre.b)));
    (void)N;
  }
  bool vec_ok(int) const { return true; }
  static const char* name() { return "EpiEncdecQF16"; }
};

// The same with the scale read from device memory (the csrc layers keep their clip values
// and the alpha derived from them on the device: csrc/kernels/cuda/cublas_wrappers.cpp:134
// CUBLASLT_POINTER_MODE_DEVICE).
struct EpiI8Dev {
  int8_t* C;
  const float* alpha;
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    const float a = alpha[0];
    if (full) {
      *reinterpret_cast<uint4*>(C + m * N + n) = requant16_packed(c, a);
      return;
    }
    int q[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) q[i] = requant_acc(c[i], a);
    store16_i8(C + m * N + n, n, N, q, full);
  }
  bool vec_ok(int N) const { return N % 16 == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0; }
  static const char* name() { return "EpiI8Dev"; }
};

// requantise to the GEMM's int8 output code, then dequant + bias + activation +
// requant exactly as the stand-alone bias/activation kernel would on that code.
template <int ACT>
struct EpiActI8 {
  int8_t* C;
  const __half* bias;
  float alpha, dequant_scale, quant_scale, clip_max;
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    float b[16];
    if (full) {  // n % 16 == 0 here, so the two 16-byte bias loads are aligned when bias is
      const half8_t b0 = *reinterpret_cast<const half8_t*>(bias + n);
      const half8_t b1 = *reinterpret_cast<const half8_t*>(bias + n + 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        b[i] = __half2float(b0.v[i]);
        b[8 + i] = __half2float(b1.v[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) b[i] = n + i < N ? __half2float(bias[n + i]) : 0.f;
    }
    int q[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      q[i] = dequant_bias_act_requant<ACT>(requant_acc(c[i], alpha), dequant_scale, b[i],
                                           quant_scale, clip_max);
    store16_i8(C + m * N + n, n, N, q, full);
  }
  bool vec_ok(int N) const {
    return N % 16 == 0 &&
           ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(bias)) & 15u) == 0;
  }
  static const char* name() { return ACT == kActGelu ? "EpiGeluI8" : "EpiReluI8"; }
};

template <int ACT>
__global__ void __launch_bounds__(256)
build_act_lut_kernel(int8_t* __restrict__ lut, const __half* __restrict__ bias, int N,
                     float dequant_scale, float quant_scale, float clip_max) {
  const int n = blockIdx.x;
  const int code = (int)threadIdx.x - 128;
  lut[(long)n * 256 + threadIdx.x] = (int8_t)dequant_bias_act_requant<ACT>(
      code, dequant_scale, __half2float(bias[n]), quant_scale, clip_max);
}

// requantise to the GEMM's int8 output code, then dequant + bias and scatter into the
// three [B, h, S, d] fp16 tensors exactly as the QKV arrange kernel would.
// Requires N == 3*h*d, d % 16 == 0.
struct EpiQkvF16 {
  __half* qkv;
  const __half* bias;
  long max_batch_dim;
  float alpha, dequant_scale;
  int seq_len, head_num, dim_per_head;
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool) const {
    const int hidden = head_num * dim_per_head;
    const int which = n / hidden, i = n - which * hidden;
    const int head = i / dim_per_head, dim = i - head * dim_per_head;
    const int b = (int)(m / seq_len), s = (int)(m - (long)b * seq_len);
    __half* dst = qkv + max_batch_dim * which +
                  (((long)b * head_num + head) * seq_len + s) * dim_per_head + dim;
    const half8_t b0 = *reinterpret_cast<const half8_t*>(bias + n);
    const half8_t b1 = *reinterpret_cast<const half8_t*>(bias + n + 8);
    half8_t lo, hi;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      lo.v[k] = __float2half_rn(dequant_add_bias_h(requant_acc(c[k], alpha), dequant_scale,
                                                   __half2float(b0.v[k])));
      hi.v[k] = __float2half_rn(dequant_add_bias_h(requant_acc(c[8 + k], alpha), dequant_scale,
                                                   __half2float(b1.v[k])));
    }
    *reinterpret_cast<half8_t*>(dst) = lo;
    *reinterpret_cast<half8_t*>(dst + 8) = hi;
    (void)N;
  }
  bool vec_ok(int) const { return true; }
  static const char* name() { return "EpiQkvF16"; }
};

// Epilogues with operands that can be requested before the product is known (decode-step
// kernel): a bias slice kept in registers, or the table rows of the workgroup's columns in LDS.
struct EpiNoPre {};
// epilogues that can store one element at a time (what the decode-step kernels use)
template <typename Epi, typename = void>
struct has_store1 : std::false_type {};
template <typename Epi>
struct has_store1<Epi, std::void_t<typename Epi::Pre1>> : std::true_type {};
template <typename Epi>
struct epi_pre {
  typedef EpiNoPre type;
  static constexpr bool value = false;
};
template <>
struct epi_pre<EpiDecQkvI8> {
  typedef EpiDecQkvI8::Pre type;
  static constexpr bool value = true;
};
template <>
struct epi_pre<EpiEncdecQF16> {
  typedef EpiEncdecQF16::Pre type;
  static constexpr bool value = true;
};

// FULL: every 16-column group of the output exists and may be stored as a vector (N % 16
// == 0 and the epilogue's alignment holds), so the scalar tail path is not even compiled:
// a kernel's instructions are fetched cold on every launch, and code that is never run
// still sits between the lines that are.
// int32 output keeps a lane's accumulators along the rows (the activation fragment is the first
// MFMA operand): register k of lane (l32, g) is row 8 (k / 4) + 4 g + k % 4 of column sigma(l32)
// of its 32 x 32 block, and a store instruction writes two whole 128-byte lines.
template <typename Epi>
constexpr bool rows_in_regs = std::is_same<Epi, EpiI32>::value;

template <typename Epi>
__device__ __forceinline__ v16i mfma_i8_tile(const v4i& w, const v4i& a, const v16i& c) {
  if constexpr (rows_in_regs<Epi>) return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, w, c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_i32_32x32x32_i8(w, a, c, 0, 0, 0);
}

template <typename Epi, int MB, int NB, bool FULL = false>
__device__ __forceinline__ void store_tile_acc(const Epi& epi, const v16i (&acc)[MB][NB], int m0,
                                               int n0, int wm, int wn, int l32, int g, int M, int N,
                                               bool vec_store, long m_off = 0) {
  if constexpr (rows_in_regs<Epi>) {
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int n = n0 + wn * (NB * 32) + j * 32 + sigma(l32);
        int32_t* cp = epi.C + n;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          const long m = m0 + wm * (MB * 32) + i * 32 + 8 * (k >> 2) + 4 * g + (k & 3);
          if (m < M && n < N) cp[(m + m_off) * N] = acc[i][j][k];
        }
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const long m = m0 + wm * (MB * 32) + i * 32 + l32;
    if (m < M) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int n = n0 + wn * (NB * 32) + j * 32 + 16 * g;
        if (n < N)
          epi.store16(m + m_off, n, N, acc[i][j], FULL ? true : (vec_store && n + 16 <= N));
      }
    }
  }
}

// linear work index -> tile.  Workgroups (and the persistent kernel's work items) are
// dealt round-robin to the 8 XCDs; renumber so that each XCD (own L2) works on a
// contiguous run of tiles, walked in column-major order of 8-tile-tall groups so that a
// run shares W columns and A rows.
// Work-item counts stay below 2^24 (checked by the dispatcher): with both operands masked to
// 24 bits the compiler divides through a float reciprocal, a dozen instructions instead of
// the forty of a full 32-bit division -- this arithmetic runs before the first load of a
// launch and sits in the kernel four times.
__device__ __forceinline__ int div24(int a, int b) {
  return (int)(((unsigned)a & 0xffffffu) / ((unsigned)b & 0xffffffu));
}
__device__ __forceinline__ void tile_of(int t, int nblk, int tiles_m, int tiles_n, int& tile_m,
                                        int& tile_n) {
  const int per = nblk / 8, rem = nblk % 8;
  const int xcd = t % 8, loc = t / 8;
  const int pid = xcd * per + (xcd < rem ? xcd : rem) + loc;
  constexpr int GROUP = 8;
  const int group_sz = GROUP * tiles_n;
  const int grp = div24(pid, group_sz);
  const int in_grp = pid - grp * group_sz;
  const int first_m = grp * GROUP;
  const int gm = min(tiles_m - first_m, GROUP);
  tile_n = div24(in_grp, gm);
  tile_m = first_m + (in_grp - tile_n * gm);
}

// ---------------------------------------------------------------------------------
// Fast path: persistent, direct-to-LDS, 3-stage ring, cross-tile prefetch, 128x64 tiles.
// Preconditions (checked by the dispatcher): K % 128 == 0, (rows-1)*K + 128 < 2^32 for
// both operands, operands 16-byte aligned.
//
// One K step = 128 bytes of K = four 32-byte slices of 2 (rows) x 1 (columns) MFMA blocks per
// wavefront.  The operand fragments of slice s + 1 are read from LDS into a second set of
// registers while the MFMAs of slice s run, and the loop turns right after the step's
// barrier: the last slice of a step is multiplied after the first fragments of the next
// step have been requested, so neither the LDS latency nor the meeting of the wavefronts
// leaves the matrix unit idle.  The barrier of step i proves that the loads of step i + 1
// have landed and that every wavefront has read all of step i; the loads of step i + 3 then
// go into the stage of step i.  72 KB of LDS: two workgroups per compute unit.  With short K
// loops (TNST = 2: 48 KB, three workgroups per compute unit, loads one step ahead) a third
// resident workgroup hides more than the deeper ring (4096 x 2304 x 768: 14.0 against 15.0 us;
// 4096 x 768 x 3072 with int32 output: 21.5 against 20.5 us).
// ---------------------------------------------------------------------------------
constexpr int kSBN = 64;  // tile width of the fast path
constexpr size_t kStreamStageBytes = (size_t)(kBM + kSBN) * kBK;

template <typename Epi, bool FULL, int TNST, bool LDSTAB = false>
__global__ void __launch_bounds__(256)
gemm_i8_stream_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi, int M,
                      int N, int K, int tiles_m, int tiles_n, bool vec_store, int ksplit) {
  constexpr int NST = TNST;  // 3: loads two K steps ahead; 2: one step ahead, 48 KB
  constexpr int STAGE = (kBM + kSBN) * kBK;      // 24 KB: A tile then W tile
  constexpr int NA = kBM / 32, NW = kSBN / 32;   // 1-KB DMA instructions per wavefront per stage
  constexpr int PER = NA + NW;
  extern __shared__ __align__(16) int8_t smem[];
  // work item = (K range, tile): with ksplit > 1 every tile is computed ksplit times over
  // disjoint K ranges and range p stores to rows [p * M, (p + 1) * M) of the output
  const int ntile = tiles_m * tiles_n;
  const int nblk = ntile * ksplit;
  const int G = gridDim.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, g = lane >> 5;
  const int my_tiles = (nblk - (int)blockIdx.x + G - 1) / G;
  const int kpart = K / ksplit;  // bytes of K per range (a multiple of kBK)
  const int nk = kpart / kBK;
  const int total_it = my_tiles * nk;

  // DMA sources: each instruction moves 8 rows x 128 B; lane i lands in LDS slot i of that
  // 1-KB block, so it fetches the chunk the swizzle puts there.  Row clamping keeps the
  // reads of partial tiles in bounds (the clamped rows are never stored).
  uint32_t a_src[NA], w_src[NW];
  auto set_src = [&](int j) {
    const int item = blockIdx.x + j * G;
    const int part = ksplit == 1 ? 0 : div24(item, ntile);
    const uint32_t koff = (uint32_t)part * (uint32_t)kpart;
    int tm, tn;
    tile_of(item - part * ntile, ntile, tiles_m, tiles_n, tm, tn);
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int row = (wave + 4 * i) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ key_act(row);
      a_src[i] = (uint32_t)min(tm * kBM + row, M - 1) * (uint32_t)K + koff + c * 16;
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int row = (wave + 4 * i) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ key_wgt(row);
      w_src[i] = (uint32_t)min(tn * kSBN + row, N - 1) * (uint32_t)K + koff + c * 16;
    }
  };
  const uint32_t lds0 =
      (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
  // Issued through inline asm so that the compiler's wait-count insertion does not see an
  // outstanding LDS write and drain vmcnt before every ds_read; the waits are explicit.
  auto dma1 = [&](const int8_t* base, uint32_t voff, uint32_t lds) {
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff),
                 "s"(base)
                 : "memory");
  };
  int p_j = 0, p_kt = 0, p_st = 0;  // prefetch cursor: work item, K step, ring slot
  auto issue_next = [&]() {
    if (p_j < my_tiles) {
      const uint32_t base = lds0 + p_st * STAGE;
#pragma unroll
      for (int i = 0; i < NA; ++i) dma1(A + p_kt * kBK, a_src[i], base + (wave + 4 * i) * 1024);
#pragma unroll
      for (int i = 0; i < NW; ++i)
        dma1(W + p_kt * kBK, w_src[i], base + kBM * kBK + (wave + 4 * i) * 1024);
      if (++p_kt == nk) {
        p_kt = 0;
        if (++p_j < my_tiles) set_src(p_j);
      }
      if (++p_st == NST) p_st = 0;
    }
  };
  // LDSTAB (the tabulated epilogue, TNST = 2): the 64 table rows of a tile's columns (16 KB)
  // are brought into LDS behind the ring while the tile's K loop runs -- four 1-KB loads per
  // wavefront, issued once every wavefront has finished the previous tile's epilogue -- and
  // the epilogue looks its bytes up there instead of in global memory.
  constexpr int NTAB = kSBN * 256 / 1024 / 4;  // table loads per wavefront and tile
  int8_t* const tab_lds = smem + NST * STAGE;
  auto issue_table = [&](int j) {
    if constexpr (LDSTAB) {
      const int item = blockIdx.x + j * G;
      const int part = ksplit == 1 ? 0 : div24(item, ntile);
      int tm, tn;
      tile_of(item - part * ntile, ntile, tiles_m, tiles_n, tm, tn);
      const long first = (long)tn * kSBN * 256, last = (long)N * 256 - 16;  // bytes of the table
#pragma unroll
      for (int i = 0; i < NTAB; ++i) {
        const int q = wave + 4 * i;
        const long off = min(first + q * 1024 + lane * 16, last);  // rows beyond N: never stored
        dma1(reinterpret_cast<const int8_t*>(epi.lut), (uint32_t)off,
             lds0 + NST * STAGE + q * 1024);
      }
    }
  };
  // at most `groups` (0 or 1) of the youngest load groups may still be in flight.  Stores of
  // an epilogue count as well and only make the wait stricter; loads complete in order.
  auto wait_groups = [&](int groups) {
    if (groups >= 1)
      __builtin_amdgcn_s_waitcnt(PER | (7 << 4) | (15 << 8));  // vmcnt(PER)
    else
      __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0)
  };

  int a_off[2], a_key[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = wm * 64 + i * 32 + l32;
    a_off[i] = row * kBK;
    a_key[i] = key_act(row);
  }
  const int w_row = wn * 32 + sigma(l32);
  const int w_off = kBM * kBK + w_row * kBK, w_key = key_wgt(w_row);
  struct Frag {
    v4i a[2], w;
  };
  auto load_frag = [&](Frag& f, const int8_t* stage, int ks) {
    const int chunk = 2 * ks + g;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      f.a[i] = *reinterpret_cast<const v4i*>(stage + a_off[i] + ((chunk ^ a_key[i]) << 4));
    f.w = *reinterpret_cast<const v4i*>(stage + w_off + ((chunk ^ w_key) << 4));
  };
  v16i acc[2][1];
  auto mma = [&](const Frag& f) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      acc[i][0] = mfma_i8_tile<Epi>(f.w, f.a[i], acc[i][0]);
  };

  if (my_tiles > 0) set_src(0);
  if (my_tiles > 0) issue_table(0);
#pragma unroll
  for (int i = 0; i < NST - 1; ++i) issue_next();
  wait_groups(min(NST - 2, total_it - 1));
  __builtin_amdgcn_s_barrier();
  Frag f0, f1;
  int st = 0, kt = 0, j = 0, tm = 0, tn = 0, part = 0;
  for (int it = 0;; ++it) {
    const int8_t* stage = smem + st * STAGE;
    if (it < total_it) {
      issue_next();  // step it + 2 into the stage step it - 1 has finished with
      load_frag(f0, stage, 0);
    }
    if (it > 0) mma(f1);  // last slice of step it - 1
    if (kt == 0) {
      if (it > 0) {
        if constexpr (LDSTAB) {
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const long m = tm * kBM + wm * 64 + i * 32 + l32;
            const int n = tn * kSBN + wn * 32 + 16 * g;
            if (m < M && n < N)
              epi.store16_lds(m + (long)part * M, n, N, acc[i][0],
                              FULL ? true : (vec_store && n + 16 <= N), tab_lds, wn * 32 + 16 * g);
          }
          // every wavefront is done with this table before the next one is loaded over it
          __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
          __builtin_amdgcn_s_barrier();
          if (it < total_it) issue_table(j);
        } else {
          store_tile_acc<Epi, 2, 1, FULL>(epi, acc, tm * kBM, tn * kSBN, wm, wn, l32, g, M, N,
                                          vec_store, (long)part * M);
        }
      }
      if (it == total_it) break;
      const int item = blockIdx.x + j * G;
      part = ksplit == 1 ? 0 : div24(item, ntile);
      tile_of(item - part * ntile, ntile, tiles_m, tiles_n, tm, tn);
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[i][0] = (v16i)0;
    }
    load_frag(f1, stage, 1);
    mma(f0);
    load_frag(f0, stage, 2);
    mma(f1);
    load_frag(f1, stage, 3);
    mma(f0);
    // step it + 1 has landed for this wavefront, and its own reads of step it are done ...
    if (LDSTAB && kt == 0 && it > 0 && nk >= 2)
      // the table loads of this tile were issued after the next step's group: they may stay in
      // flight (loads complete in order), the second step's wait then covers them
      __builtin_amdgcn_s_waitcnt(NTAB | (7 << 4) | (15 << 8));  // vmcnt(NTAB)
    else
      wait_groups(min(NST - 2, total_it - 2 - it));
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    // ... and for everyone
    __builtin_amdgcn_s_barrier();
    if (++st == NST) st = 0;
    if (++kt == nk) {
      kt = 0;
      ++j;
    }
  }
  __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));
}

// The earlier form of the fast path: 128x128 tiles (2x2 MFMA blocks per wavefront), 2-stage
// ring, all fragments of a step read before its MFMAs.  Kept for the epilogues that load
// (activation tables, bias): their loads are younger than the operand groups in flight, so
// waiting for them drains the ring at every tile boundary, and this form has half as many
// boundaries (same box, FFN1 of BERT-base with the tabulated GELU: 22.6 us here, 24.5 us with
// the 128x64 kernel; the other three products of the layer are 1-2 us faster there).
template <typename Epi, bool FULL>
__global__ void __launch_bounds__(256)
gemm_i8_stream128_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi, int M,
                      int N, int K, int tiles_m, int tiles_n, bool vec_store, int ksplit) {
  constexpr int NST = 2;
  constexpr int STAGE = (kBM + kBN) * kBK;  // 32 KB: A tile then W tile
  constexpr int NA = kBM / 32, NW = kBN / 32;  // 1-KB DMA instructions per wavefront per stage
  extern __shared__ __align__(16) int8_t smem[];
  // work item = (K range, tile): with ksplit > 1 every tile is computed ksplit times over
  // disjoint K ranges and range p stores to rows [p * M, (p + 1) * M) of the output
  const int ntile = tiles_m * tiles_n;
  const int nblk = ntile * ksplit;
  const int G = gridDim.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, g = lane >> 5;
  const int my_tiles = (nblk - (int)blockIdx.x + G - 1) / G;
  const int kpart = K / ksplit;  // bytes of K per range (a multiple of kBK)
  const int nk = kpart / kBK;

  // DMA sources: each instruction moves 8 rows x 128 B; lane i lands in LDS slot i of that
  // 1-KB block, so it fetches the chunk the swizzle puts there.  Row clamping keeps the
  // reads of partial tiles in bounds (the clamped rows are never stored).
  uint32_t a_src[NA], w_src[NW];
  auto set_src = [&](int j) {
    const int item = blockIdx.x + j * G;
    const int part = ksplit == 1 ? 0 : div24(item, ntile);
    const uint32_t koff = (uint32_t)part * (uint32_t)kpart;
    int tm, tn;
    tile_of(item - part * ntile, ntile, tiles_m, tiles_n, tm, tn);
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int row = (wave + 4 * i) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ key_act(row);
      a_src[i] = (uint32_t)min(tm * kBM + row, M - 1) * (uint32_t)K + koff + c * 16;
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int row = (wave + 4 * i) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ key_wgt(row);
      w_src[i] = (uint32_t)min(tn * kBN + row, N - 1) * (uint32_t)K + koff + c * 16;
    }
  };
  const uint32_t lds0 =
      (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
  // Issued through inline asm so that the compiler's wait-count insertion does not see an
  // outstanding LDS write and drain vmcnt before every ds_read; the waits are explicit.
  auto dma1 = [&](const int8_t* base, uint32_t voff, uint32_t lds) {
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff),
                 "s"(base)
                 : "memory");
  };
  int p_j = 0, p_kt = 0, p_st = 0;  // prefetch cursor: tile, K step, ring slot
  auto issue_next = [&]() {
    if (p_j < my_tiles) {
      const uint32_t base = lds0 + p_st * STAGE;
#pragma unroll
      for (int i = 0; i < NA; ++i) dma1(A + p_kt * kBK, a_src[i], base + (wave + 4 * i) * 1024);
#pragma unroll
      for (int i = 0; i < NW; ++i)
        dma1(W + p_kt * kBK, w_src[i], base + kBM * kBK + (wave + 4 * i) * 1024);
      if (++p_kt == nk) {
        p_kt = 0;
        if (++p_j < my_tiles) set_src(p_j);
      }
      p_st ^= 1;
    }
  };

  int a_off[2], w_off[2], a_key[2], w_key[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = wm * 64 + i * 32 + l32;
    a_off[i] = row * kBK;
    a_key[i] = key_act(row);
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = wn * 64 + j * 32 + sigma(l32);
    w_off[j] = kBM * kBK + row * kBK;
    w_key[j] = key_wgt(row);
  }

  if (my_tiles > 0) set_src(0);
  issue_next();
  int st = 0;
  for (int j = 0; j < my_tiles; ++j) {
    const int item = blockIdx.x + j * G;
    const int part = ksplit == 1 ? 0 : div24(item, ntile);
    int tm, tn;
    tile_of(item - part * ntile, ntile, tiles_m, tiles_n, tm, tn);
    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) acc[i][jj] = (v16i)0;
    for (int kt = 0; kt < nk; ++kt) {
      // stage `st` has landed for this wavefront ...
      __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // vmcnt(0)
      // ... and for everyone; everyone is also done reading the other stage
      __builtin_amdgcn_s_barrier();
      issue_next();
      const int8_t* stage = smem + st * STAGE;
      v4i bv[kBK / 32][2], av[kBK / 32][2];
#pragma unroll
      for (int ks = 0; ks < kBK / 32; ++ks) {
        const int chunk = 2 * ks + g;
#pragma unroll
        for (int i = 0; i < 2; ++i)
          bv[ks][i] = *reinterpret_cast<const v4i*>(stage + a_off[i] + ((chunk ^ a_key[i]) << 4));
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
          av[ks][jj] = *reinterpret_cast<const v4i*>(stage + w_off[jj] + ((chunk ^ w_key[jj]) << 4));
      }
#pragma unroll
      for (int ks = 0; ks < kBK / 32; ++ks)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj)
            acc[i][jj] = mfma_i8_tile<Epi>(av[ks][jj], bv[ks][i], acc[i][jj]);
      st ^= 1;
    }
    store_tile_acc<Epi, 2, 2, FULL>(epi, acc, tm * kBM, tn * kBN, wm, wn, l32, g, M, N, vec_store,
                                    (long)part * M);
  }
  __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));
}

// ---------------------------------------------------------------------------------
// Wide-tile path: one large output tile per workgroup, for products with enough of them to
// give every compute unit one (M and N in the thousands).
//
// What the measurements on this part say: under int8 MFMA load the shader clock sits near
// 1.6 GHz (of 2.4), a kernel's stores cost their bytes / ~4.7 TB/s after its last wavefront
// has finished (the write-back of the XCD's L2 at the kernel boundary), a launch needs
// ~1.3 us before its first operands have landed (the L2 starts cold), and one wavefront per
// SIMD keeps the matrix unit ~2/3 busy where two keep it ~95 % busy.  So: 8 wavefronts (two
// per SIMD) share one 256 x 192 / 256 x 256 / 256 x 128 tile -- operand bytes per MFMA fall
// with the tile area per compute unit, which is what both the 64 B/clk global->LDS path and
// the LDS port are short of -- with 64 x 96 / 128 x 64 / 64 x 64 wavefront tiles; K steps of
// 128 bytes go through a ring of NST stages filled by global_load_lds_dwordx4; fragments are
// double-buffered per 32-byte slice and the issue order inside a slice is pinned (one LDS
// read after each of the first MFMAs).  The step's barrier sits before the last slice's
// MFMAs; after it the freed stage is refilled with step kt + NST.
// The tabulated epilogue brings its TN x 256-byte table into the stage that the
// second-to-last step frees, while the last step is multiplied.
// Preconditions (checked by the dispatcher): K % 128 == 0, K / 128 >= NST, N % 16 == 0 and the
// epilogue's vector path legal, 32-bit operand offsets, operands 16-byte aligned.
// ---------------------------------------------------------------------------------
template <typename Epi, int WGM, int WGN, int MB, int NB, int NST>
__global__ void __launch_bounds__(64 * WGM * WGN)
gemm_i8_tile_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi, int M,
                    int N, int K, int tiles_m, int tiles_n, bool, int) {
  extern __shared__ __align__(16) int8_t smem[];
  // the operand pointers are wanted in registers here, so that their kernel-argument load
  // leaves with the one for the shape instead of after the tile arithmetic that needs the shape
  // (the tile arithmetic below is made to wait for them)
  asm volatile("" : "+s"(tiles_m) : "s"(A), "s"(W));
  constexpr int TM = WGM * MB * 32;
  int tm, tn;
  tile_of(blockIdx.x, tiles_m * tiles_n, tiles_m, tiles_n, tm, tn);
  tile_gemm<Epi, WGM, WGN, MB, NB, NST>(A, W, epi, tm * TM, M, N, K, tn, smem);
}

// ---------------------------------------------------------------------------------
// Generic path: register-staged double buffering, zero-filled tails.
// ---------------------------------------------------------------------------------
template <int ROWS>
__device__ __forceinline__ void load_tile(const int8_t* __restrict__ base, int row0, int nrows,
                                          int K, int k0, int tid, v4i (&regs)[ROWS / 32]) {
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i) {
    const int row = (tid >> 3) + 32 * i;
    const int kc = k0 + (tid & 7) * 16;
    const int grow = row0 + row;
    if (grow < nrows && kc < K)
      regs[i] = *reinterpret_cast<const v4i*>(base + (long)grow * K + kc);
    else
      regs[i] = (v4i)0;
  }
}

template <int ROWS, bool WGT>
__device__ __forceinline__ void store_tile(int8_t* lds, int tid, const v4i (&regs)[ROWS / 32]) {
#pragma unroll
  for (int i = 0; i < ROWS / 32; ++i) {
    const int row = (tid >> 3) + 32 * i;
    const int key = WGT ? key_wgt(row) : key_act(row);
    *reinterpret_cast<v4i*>(lds + row * kBK + (((tid & 7) ^ key) << 4)) = regs[i];
  }
}

template <typename Epi>
__global__ void __launch_bounds__(256)
gemm_i8_generic_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi, int M,
                       int N, int K, int tiles_m, int tiles_n, bool vec_store, int) {
  constexpr int kStage = (kBM + kBN) * kBK;
  extern __shared__ __align__(16) int8_t smem[];
  int tile_m, tile_n;
  tile_of(blockIdx.x, tiles_m * tiles_n, tiles_m, tiles_n, tile_m, tile_n);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int m0 = tile_m * kBM, n0 = tile_n * kBN;

  v16i acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = (v16i)0;

  v4i ra[kBM / 32], rw[kBN / 32];
  const int nk = (K + kBK - 1) / kBK;
  load_tile<kBM>(A, m0, M, K, 0, tid, ra);
  load_tile<kBN>(W, n0, N, K, 0, tid, rw);
  store_tile<kBM, false>(smem, tid, ra);
  store_tile<kBN, true>(smem + kBM * kBK, tid, rw);
  __syncthreads();

  int a_off[2], w_off[2], a_key[2], w_key[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = wm * 64 + i * 32 + l32;
    a_off[i] = row * kBK;
    a_key[i] = key_act(row);
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = wn * 64 + j * 32 + sigma(l32);
    w_off[j] = row * kBK;
    w_key[j] = key_wgt(row);
  }

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      load_tile<kBM>(A, m0, M, K, (kt + 1) * kBK, tid, ra);
      load_tile<kBN>(W, n0, N, K, (kt + 1) * kBK, tid, rw);
    }
    const int8_t* pa = smem + cur * kStage;
    const int8_t* pw = pa + kBM * kBK;
#pragma unroll
    for (int ks = 0; ks < kBK / 32; ++ks) {
      const int chunk = 2 * ks + g;
      v4i bv[2], av[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        bv[i] = *reinterpret_cast<const v4i*>(pa + a_off[i] + ((chunk ^ a_key[i]) << 4));
#pragma unroll
      for (int j = 0; j < 2; ++j)
        av[j] = *reinterpret_cast<const v4i*>(pw + w_off[j] + ((chunk ^ w_key[j]) << 4));
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = mfma_i8_tile<Epi>(av[j], bv[i], acc[i][j]);
    }
    if (kt + 1 < nk) {
      int8_t* nxt = smem + (cur ^ 1) * kStage;
      store_tile<kBM, false>(nxt, tid, ra);
      store_tile<kBN, true>(nxt + kBM * kBK, tid, rw);
    }
    __syncthreads();
  }
  store_tile_acc<Epi, 2, 2>(epi, acc, m0, n0, wm, wn, l32, g, M, N, vec_store);
}

// ---------------------------------------------------------------------------------
// Decode-step path: M <= 64 rows (batch x beam of one generation step).  The product is
// bound by streaming the weight matrix once from HBM, so the kernel is organised around
// that stream: one workgroup owns 32 output columns (32 weight rows of K bytes, a contiguous
// slab), its 4 wavefronts take the 128-byte K chunks round-robin, and every lane loads its
// MFMA operands straight from global memory -- 64 contiguous bytes of one weight row per
// chunk -- with all loads of a chunk pair in flight before the MFMAs.  There is no LDS
// staging (each weight byte is used by exactly one wavefront) and no tile loop; the partial
// accumulators of the 4 wavefronts meet in LDS and go through the same epilogues.
// Preconditions: K % 128 == 0, operands 16-byte aligned.
// ---------------------------------------------------------------------------------
template <typename Epi, int MBLK, bool FULL>
__global__ void __launch_bounds__(256)
gemm_i8_skinny_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi, int M,
                      int N, int K, int, int, bool vec_store, int ksplit) {
  __shared__ int red[4][MBLK][16][64];  // [wavefront][m block][register][lane]
  constexpr bool kLut = std::is_same<Epi, EpiLutI8>::value;
  __shared__ __align__(16) int8_t tab[kLut ? 32 * 256 : 16];  // table rows of the 32 columns
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  // blockIdx.x = column block + (K range) * column blocks; range p stores to rows
  // [p * M, (p + 1) * M) of the output
  const int ncol = (int)gridDim.x / ksplit;
  const int part = (int)blockIdx.x / ncol;
  const int n0 = ((int)blockIdx.x % ncol) * 32;
  // What the epilogue reads besides the product is requested first, so that it travels with
  // the weights instead of after the last matrix instruction: the bias slice of the lane's 16
  // columns, or 32 bytes per thread of the 32 table rows (columns past N clamped).
  typename epi_pre<Epi>::type pre;
  if constexpr (epi_pre<Epi>::value) pre = epi.prefetch(max(min(n0 + 16 * g, N - 16), 0));
  uint4 tab0, tab1;
  if constexpr (kLut) {
    const int8_t* tp = epi_lut(epi) + (long)min(n0 + (tid >> 3), N - 1) * 256 + (tid & 7) * 32;
    tab0 = *reinterpret_cast<const uint4*>(tp);
    tab1 = *reinterpret_cast<const uint4*>(tp + 16);
  }
  const int8_t* wp = W + (long)min(n0 + sigma(l32), N - 1) * K + g * 64;
  const int8_t* ap[MBLK];
#pragma unroll
  for (int i = 0; i < MBLK; ++i) ap[i] = A + (long)min(i * 32 + l32, M - 1) * K + g * 64;
  v16i acc[MBLK];
#pragma unroll
  for (int i = 0; i < MBLK; ++i) acc[i] = (v16i)0;
  const int nch_part = K / kBK / ksplit;
  const int nch = (part + 1) * nch_part;
  for (int ch = part * nch_part + wave; ch < nch; ch += 8) {
    const int k0 = ch * kBK;
    const bool two = ch + 4 < nch;
    const int k1 = two ? k0 + 4 * kBK : k0;
    v4i wv[2][4], av[2][MBLK][4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      wv[0][ks] = *reinterpret_cast<const v4i*>(wp + k0 + ks * 16);
      wv[1][ks] = *reinterpret_cast<const v4i*>(wp + k1 + ks * 16);
    }
#pragma unroll
    for (int i = 0; i < MBLK; ++i)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        av[0][i][ks] = *reinterpret_cast<const v4i*>(ap[i] + k0 + ks * 16);
        av[1][i][ks] = *reinterpret_cast<const v4i*>(ap[i] + k1 + ks * 16);
      }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < MBLK; ++i)
        acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wv[0][ks], av[0][i][ks], acc[i], 0, 0, 0);
    if (two) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int i = 0; i < MBLK; ++i)
          acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wv[1][ks], av[1][i][ks], acc[i], 0, 0, 0);
    }
  }
#pragma unroll
  for (int i = 0; i < MBLK; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) red[wave][i][r][lane] = acc[i][r];
  if constexpr (kLut) {
    *reinterpret_cast<uint4*>(tab + (tid >> 3) * 256 + (tid & 7) * 32) = tab0;
    *reinterpret_cast<uint4*>(tab + (tid >> 3) * 256 + (tid & 7) * 32 + 16) = tab1;
  }
  __syncthreads();
  if (wave < MBLK) {
    v16i c;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      c[r] = (red[0][wave][r][lane] + red[1][wave][r][lane]) +
             (red[2][wave][r][lane] + red[3][wave][r][lane]);
    const long m = wave * 32 + l32;
    const int n = n0 + 16 * g;
    if (m < M && n < N) {
      const bool full = FULL ? true : (vec_store && n + 16 <= N);
      if constexpr (kLut)
        epi.store16_lds(m + (long)part * M, n, N, c, full, tab, 16 * g);
      else if constexpr (epi_pre<Epi>::value)
        epi.store16_pre(m + (long)part * M, n, N, c, full, pre);
      else
        epi.store16(m + (long)part * M, n, N, c, full);
    }
  }
}

// ---------------------------------------------------------------------------------
// Decode-step path on 16 x 16 x 64 products (K range of a workgroup a multiple of 256 bytes).
// The 32 x 32 x 32 form above gives a lane one weight row, so a load instruction of a
// wavefront touches 64 different 64-byte segments and uses 16 bytes of each: the address unit
// of the compute unit, not memory, bounds it (measured: 3.4 us from the first instruction to
// the last product of a 32 KB slab).  With 16 x 16 x 64 products the four lanes l, l + 16,
// l + 32, l + 48 hold the four 16-byte quarters of one row's 64-byte K slice, so an
// instruction reads 16 whole segments, and 16 activation rows -- one decoding batch -- fill
// the product with nothing clamped.  A workgroup still owns 32 output columns (two 16-column
// blocks) for all rows; wavefront w takes the w-th quarter of the workgroup's K range, four
// slices per round, every load of a round requested before its first product; the partial
// tiles meet in LDS, where the epilogue threads (one per row and column block) gather the 16
// columns the epilogues expect.
// ---------------------------------------------------------------------------------
template <typename Epi, int MB, bool FULL, int NB = 2>
__global__ void __launch_bounds__(256)
gemm_i8_skinny16_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi, int M,
                        int N, int K, int kw, int, bool vec_store, int) {
  // NB 16-column blocks per workgroup: 2, or 1 where that still fits one round of the chip
  __shared__ int red[4][MB][NB][4][64];  // [wavefront][row block][column block][register][lane]
  constexpr bool kLut = std::is_same<Epi, EpiLutI8>::value;
  __shared__ __align__(16) int8_t tab[kLut ? 16 * NB * 256 : 16];  // table rows of the columns
  asm volatile("" ::"s"(A), "s"(W));  // one batch of kernel-argument loads, not two in a row
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kq = lane >> 4;
  // grid: x = column block, y = K range (plane of the output); kw = bytes of K per wavefront,
  // a multiple of 64, from the host: a kernel of a few microseconds cannot afford integer
  // divisions and kernel-argument loads that wait for one another before its first load
  const int part = (int)blockIdx.y;
  const int n0 = (int)blockIdx.x * (16 * NB);
  // grid z: blocks of 16 MB rows (more than 32 rows run as two workgroups of 32 rows per column
  // block: half the fragments and products in a row for each, the weights read twice from L2)
  const int m0 = (int)blockIdx.z * (16 * MB);
  // epilogue thread t: row t % (16 MB), column block t / (16 MB) (threads beyond 32 MB idle)
  const int em = tid % (16 * MB), eblk = (tid / (16 * MB)) & (NB - 1);
  // What the epilogue reads besides the product travels with the weights.
  constexpr bool kOne = has_store1<Epi>::value;  // every thread stores one element per block
  const int ecol = tid & 15, erow = tid >> 4;    // ... element (erow, ecol) of a 16 x 16 block
  typename epi_pre<Epi>::type pre;
  typename std::conditional<kOne, Epi, EpiI32>::type::Pre1 pre1[NB];
  if constexpr (kOne) {
#pragma unroll
    for (int b = 0; b < NB; ++b) pre1[b] = epi.prefetch1(min(n0 + 16 * b + ecol, N - 1));
  } else if constexpr (epi_pre<Epi>::value) {
    pre = epi.prefetch(max(min(n0 + 16 * eblk, N - 16), 0));
  }
  uint4 tab0, tab1;
  if constexpr (kLut) {
    const int8_t* tp = epi_lut(epi) + (long)min(n0 + ((tid >> 3) & (16 * NB - 1)), N - 1) * 256 + (tid & 7) * 32;
    tab0 = *reinterpret_cast<const uint4*>(tp);
    tab1 = *reinterpret_cast<const uint4*>(tp + 16);
  }
  const long kbase = ((long)part * 4 + wave) * kw + kq * 16;
  const int8_t* wp[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) wp[b] = W + (long)min(n0 + 16 * b + l16, N - 1) * K + kbase;
  const int8_t* ap[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i) ap[i] = A + (long)min(m0 + 16 * i + l16, M - 1) * K + kbase;
  v4i acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[i][b] = (v4i)0;
  const int ns = kw / 64;
  for (int s0 = 0; s0 < ns; s0 += 4) {
    v4i wv[4][NB], av[4][MB];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int off = min(s0 + u, ns - 1) * 64;  // clamped: the loads stay unconditional
#pragma unroll
      for (int b = 0; b < NB; ++b) wv[u][b] = *reinterpret_cast<const v4i*>(wp[b] + off);
#pragma unroll
      for (int i = 0; i < MB; ++i) av[u][i] = *reinterpret_cast<const v4i*>(ap[i] + off);
    }
    // Every load of the round stays ahead of its first product: a slice whose products are
    // conditional (a K range of fewer than four slices) had its loads moved into that branch by
    // the compiler, behind the wait for the others -- a second trip to memory in a kernel of
    // one.  The scheduling barrier keeps the requests together, the empty statements keep the
    // fragments live whatever the branch does.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int b = 0; b < NB; ++b) asm volatile("" : "+v"(wv[u][b]));
#pragma unroll
      for (int i = 0; i < MB; ++i) asm volatile("" : "+v"(av[u][i]));
      if (s0 + u < ns) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
          for (int b = 0; b < NB; ++b)
            acc[i][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[u][b], av[u][i], acc[i][b], 0, 0, 0);
      }
    }
  }
  // lane holds C[row 16 i + l16][column n0 + 16 b + 4 kq + r], r = 0..3
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][i][b][r][lane] = acc[i][b][r];
  if constexpr (kLut) {
    if (tid < 128 * NB) {
      *reinterpret_cast<uint4*>(tab + (tid >> 3) * 256 + (tid & 7) * 32) = tab0;
      *reinterpret_cast<uint4*>(tab + (tid >> 3) * 256 + (tid & 7) * 32 + 16) = tab1;
    }
  }
  __syncthreads();
  if constexpr (kOne) {
    // A wavefront that walks 16 columns of a row in a row of instructions runs as long as the
    // rest of the kernel: the instructions of one wavefront, not the memory, bound a launch of
    // this size.  So every thread finishes one element of each 16 x 16 block: four LDS reads,
    // three adds, the epilogue of one value, one store; 16 lanes write 16 neighbouring columns.
    const int src = (ecol >> 2) * 16 + erow, r = ecol & 3;  // lane and register that held it
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int n = n0 + 16 * b + ecol;
      const auto blk = epi.block1(min(n, N - 1));  // what the elements of the column share
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        const int m = m0 + 16 * i + erow;
        if (m < M && n < N) {
          const int acc = (red[0][i][b][r][src] + red[1][i][b][r][src]) +
                          (red[2][i][b][r][src] + red[3][i][b][r][src]);
          epi.store1(m + (long)part * M, blk, N, acc, pre1[b], tab, 16 * b + ecol);
        }
      }
    }
  } else if (tid < 16 * NB * MB) {
    const int n = n0 + 16 * eblk;
    if (m0 + em < M && n < N) {
      v16i c;
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int src = q * 16 + (em & 15);
          c[4 * q + r] = (red[0][em >> 4][eblk][r][src] + red[1][em >> 4][eblk][r][src]) +
                         (red[2][em >> 4][eblk][r][src] + red[3][em >> 4][eblk][r][src]);
        }
      const bool full = FULL ? true : (vec_store && n + 16 <= N);
      if constexpr (kLut)
        epi.store16_lds(m0 + em + (long)part * M, n, N, c, full, tab, 16 * eblk);
      else if constexpr (epi_pre<Epi>::value)
        epi.store16_pre(m0 + em + (long)part * M, n, N, c, full, pre);
      else
        epi.store16(m0 + em + (long)part * M, n, N, c, full);
    }
  }
}

// The same for outputs of thousands of columns (vocabulary logits), K <= 1024, no K split: with
// 32 columns per workgroup such a product is a thousand workgroups that each wait for their
// own memory round trip, several rounds of the chip; here a workgroup walks NPAIR pairs of
// 16-column blocks with its activation fragments resident in registers (fetched once), the
// weights of the next pair requested before the products of the current one, and the partial
// tiles of consecutive pairs in alternating LDS buffers (one barrier per pair).
template <typename Epi, int MB, int NPAIR>
__global__ void __launch_bounds__(256)
gemm_i8_skinny16_wide_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi,
                             int M, int N, int K, int kw, int, bool vec_store, int) {
  __shared__ int red[2][4][MB][2][4][64];
  asm volatile("" ::"s"(A), "s"(W));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kq = lane >> 4;
  const int n00 = (int)blockIdx.x * (32 * NPAIR);
  const int em = tid % (16 * MB), eblk = (tid / (16 * MB)) & 1;
  const long kbase = (long)wave * kw + kq * 16;
  const int ns = kw / 64;  // 1 .. 4 slices per wavefront
  v4i av[4][MB];
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int i = 0; i < MB; ++i)
      av[u][i] = *reinterpret_cast<const v4i*>(A + (long)min(16 * i + l16, M - 1) * K + kbase +
                                               min(u, ns - 1) * 64);
  auto load_w = [&](int pair, v4i (&wv)[4][2]) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int8_t* wp = W + (long)min(n00 + 32 * pair + 16 * b + l16, N - 1) * K + kbase;
#pragma unroll
      for (int u = 0; u < 4; ++u) wv[u][b] = *reinterpret_cast<const v4i*>(wp + min(u, ns - 1) * 64);
    }
  };
  v4i wv[2][4][2];
  load_w(0, wv[0]);
#pragma unroll
  for (int pair = 0; pair < NPAIR; ++pair) {
    if (n00 + 32 * pair >= N) break;  // (uniform)
    if (pair + 1 < NPAIR) load_w(pair + 1, wv[(pair + 1) & 1]);
    v4i acc[MB][2];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int b = 0; b < 2; ++b) acc[i][b] = (v4i)0;
    __builtin_amdgcn_sched_barrier(0);  // (the requests stay ahead of the products, see above)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int b = 0; b < 2; ++b) asm volatile("" : "+v"(wv[pair & 1][u][b]));
      if (pair == 0) {
#pragma unroll
        for (int i = 0; i < MB; ++i) asm volatile("" : "+v"(av[u][i]));
      }
      if (u < ns) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
          for (int b = 0; b < 2; ++b)
            acc[i][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[pair & 1][u][b], av[u][i],
                                                              acc[i][b], 0, 0, 0);
      }
    }
    auto& rd = red[pair & 1];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) rd[wave][i][b][r][lane] = acc[i][b][r];
    __syncthreads();
    if constexpr (has_store1<Epi>::value && MB <= 2) {
      // one element per thread and 16 x 16 block (see gemm_i8_skinny16_kernel; with 64 rows
      // that is eight elements per thread and pair, no shorter than 16 in half the threads)
      const int ecol = tid & 15, erow = tid >> 4;
      const int src = (ecol >> 2) * 16 + erow, r = ecol & 3;
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int n = n00 + 32 * pair + 16 * b + ecol;
        const auto blk = epi.block1(min(n, N - 1));
#pragma unroll
        for (int i = 0; i < MB; ++i) {
          const int m = 16 * i + erow;
          if (m < M && n < N) {
            const int acc1 = (rd[0][i][b][r][src] + rd[1][i][b][r][src]) +
                             (rd[2][i][b][r][src] + rd[3][i][b][r][src]);
            epi.store1(m, blk, N, acc1, typename Epi::Pre1{}, nullptr, 0);
          }
        }
      }
    } else if (tid < 32 * MB) {
      const int n = n00 + 32 * pair + 16 * eblk;
      if (em < M && n < N) {
        v16i c;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int src = q * 16 + (em & 15);
            c[4 * q + r] = (rd[0][em >> 4][eblk][r][src] + rd[1][em >> 4][eblk][r][src]) +
                           (rd[2][em >> 4][eblk][r][src] + rd[3][em >> 4][eblk][r][src]);
          }
        epi.store16(em, n, N, c, vec_store && n + 16 <= N);
      }
    }
  }
}

// ---------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------
static thread_local hipEvent_t g_ev_start = nullptr, g_ev_stop = nullptr;
// switch for A/B measurements of the one-tile-per-workgroup kernel against the persistent ones
static std::atomic<bool> g_tile_kernel_enabled{true};
// the same for the two decode-step kernels (tests compare them bit for bit)
static std::atomic<bool> g_skinny16_enabled{true};
static std::atomic<unsigned long> g_route_epoch{0};

unsigned long route_epoch() { return g_route_epoch.load(std::memory_order_acquire); }
void route_epoch_bump() { g_route_epoch.fetch_add(1, std::memory_order_acq_rel); }

void gemm_i8_time_next_launch(hipEvent_t start, hipEvent_t stop) {
  g_ev_start = start;
  g_ev_stop = stop;
}

// Compute units of the current device (256 on MI355X), read once per device: the choices below
// reason in rounds of the chip -- one, two or three resident workgroups per compute unit.
int cu_count() {
  static std::mutex mu;
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  std::lock_guard<std::mutex> lock(mu);
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

static bool stream_ok(int M, int N, int K) {
  if (K % kBK != 0) return false;
  const unsigned long long lim = 0xffffffffull;
  return (unsigned long long)M * K < lim && (unsigned long long)N * K < lim;
}

// The dynamic-LDS limit of a kernel function is raised once per device, under a lock, the
// first time that function is launched there (a function's LDS size is fixed by its template
// parameters).
template <auto Kern>
static int raise_lds_limit(size_t smem) {
  static std::mutex mu;
  static unsigned long long done = 0;  // bit per device index
  int dev = 0;
  if (int rc = lsh_check_hip(hipGetDevice(&dev), "hipGetDevice(gemm_i8)")) return rc;
  if (dev < 0 || dev >= 64) return lsh_fail(LSH_ERR_UNSUPPORTED, "int8 gemm: device index out of range");
  std::lock_guard<std::mutex> lock(mu);
  if (!(done >> dev & 1ull)) {
    if (smem > 0) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if (e != hipSuccess) return lsh_check_hip(e, "hipFuncSetAttribute(gemm_i8)");
    }
    done |= 1ull << dev;
  }
  return LSH_OK;
}

template <auto Kern, typename Epi>
static int launch(int grid, int threads, size_t smem, const int8_t* A, const int8_t* W, Epi epi,
                  int M, int N, int K, int tiles_m, int tiles_n, bool vec_store, hipStream_t s,
                  int ksplit = 1, int grid_y = 1, int grid_z = 1) {
  if (int rc = raise_lds_limit<Kern>(smem)) return rc;
  if (g_ev_start != nullptr) {
    // kernel-exact begin/end timestamps on the launch stream
    hipEvent_t e0 = g_ev_start, e1 = g_ev_stop;
    g_ev_start = g_ev_stop = nullptr;
    hipExtLaunchKernelGGL(Kern, dim3(grid, grid_y, grid_z), dim3(threads), (unsigned)smem, s, e0, e1, 0, A,
                          W, epi, M, N, K, tiles_m, tiles_n, vec_store, ksplit);
  } else {
    Kern<<<dim3(grid, grid_y, grid_z), threads, smem, s>>>(A, W, epi, M, N, K, tiles_m, tiles_n, vec_store,
                                                   ksplit);
  }
  return lsh_check_launch("gemm_i8_kernel");
}

// The 128x64 kernel wins where a tile's K loop is long against its boundary (epilogue, restart
// of the fragment pipeline), where 128x128 tiles would leave compute units without one, and
// where the half-size tiles fill the last round of the 512 resident workgroups better; with
// short K loops and whole rounds of tiles the wide form has half as many boundaries to pay
// (4096 x 4096 x 1024, int8 out: 26.3 us wide, 31.0 us narrow; 4096 x 768 x 3072: 21.8 and 20.0;
// 4096 x 2304 x 768: 15.8 and 15.3).
static bool narrow_pays(int M, int N, int K, int ksplit) {
  const long wide_items = (long)((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN) * ksplit;
  const long cus = cu_count(), res2 = 2 * cus;  // two resident workgroups per compute unit
  const long rounds_wide = (wide_items + res2 - 1) / res2,
             half_rounds_narrow = (2 * wide_items + res2 - 1) / res2;
  return K / ksplit / kBK >= 12 || wide_items < cus || half_rounds_narrow < 2 * rounds_wide;
}

// Epilogues that run the 128x128 form of the fast path: every one that reads memory (tables,
// bias vectors, a scale kept in device memory)
template <typename Epi>
struct wide_tiles : std::true_type {};
template <>
struct wide_tiles<EpiI32> : std::false_type {};
template <>
struct wide_tiles<EpiI8> : std::false_type {};

// Epilogues compiled for the one-tile-per-workgroup kernel (the products of a whole batch);
// the two decode-step epilogues only ever see M <= 64.
template <typename Epi>
struct has_tile_kernel : std::true_type {};
template <>
struct has_tile_kernel<EpiDecQkvI8> : std::false_type {};
template <>
struct has_tile_kernel<EpiEncdecQF16> : std::false_type {};

// Tile shapes of gemm_i8_tile_kernel: 8 wavefronts and a 2-stage ring (3 for 256 x 128); 128 x 96 on
// 4 wavefronts for outputs as narrow as the hidden size.
enum TileShape { kTileNone = 0, kTile256x256, kTile256x192, kTile256x128, kTile128x96 };
struct TileChoice {
  TileShape shape;
  int tm, tn;
};
// One workgroup per compute unit and round: the cost of a shape is its number of rounds times
// the tile area, plus the operand bytes a tile streams per K byte (rows + columns), which is
// what separates shapes of equal area.  Shapes that would leave more than a quarter of the
// 256 compute units without a tile in the last round, or give fewer than 128 tiles, are left to
// the persistent kernels.
static TileChoice choose_tile(int M, int N, int K) {
  TileChoice best{kTileNone, 0, 0};
  const long cus = cu_count();
  if (K % kBK != 0 || K / kBK < 3 || M < 1024) return best;
  if (N < 1024) {
    // narrow outputs (N = hidden size): 128 x 96 tiles on 4 wavefronts (32 x 96 each) when they
    // give about one tile per compute unit; measured 4096 x 768 x 768 5.8 us against 9.5 us and
    // 4096 x 768 x 3072 (int32 out) 18.3 us against 20.1 us for the persistent kernels
    const long tiles = (long)((M + 127) / 128) * ((N + 95) / 96);
    if (N % 96 == 0 && tiles >= cus * 3 / 4 && tiles <= cus) best = TileChoice{kTile128x96, 128, 96};
    return best;
  }
  const struct {
    TileShape shape;
    int tm, tn;
  } cand[] = {{kTile256x256, 256, 256}, {kTile256x192, 256, 192}, {kTile256x128, 256, 128}};
  double best_cost = 0;
  for (const auto& c : cand) {
    const long tiles = (long)((M + c.tm - 1) / c.tm) * ((N + c.tn - 1) / c.tn);
    if (tiles < cus / 2) continue;
    const long rounds = (tiles + cus - 1) / cus;
    const long last = tiles - (rounds - 1) * cus;
    if (last < cus * 9 / 16) continue;
    // wasted columns / rows of partial tiles count through the padded area
    const double area = (double)c.tm * c.tn;
    const double cost = rounds * area * (1.0 + 48.0 * (c.tm + c.tn) / area);
    if (best.shape == kTileNone || cost < best_cost) {
      best = TileChoice{c.shape, c.tm, c.tn};
      best_cost = cost;
    }
  }
  return best;
}

template <typename Epi>
static int dispatch(const int8_t* A, const int8_t* W, Epi epi, int M, int N, int K,
                    hipStream_t s, int ksplit = 1) {
  if (M <= 0 || N <= 0 || K <= 0 || !A || !W)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm: bad arguments");
  if (K % 16 != 0) return lsh_fail(LSH_ERR_UNSUPPORTED, "int8 gemm: K must be a multiple of 16");
  if (((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm: operands must be 16-byte aligned");
  const bool vec_store = epi.vec_ok(N);
  // 128 x 64 tiles in the fast path, 128 x 128 in its wide form and in the generic kernel
  const bool stream = stream_ok(M, N, K);
  const bool narrow = stream && !wide_tiles<Epi>::value && narrow_pays(M, N, K, ksplit);
  const int tiles_m = (M + kBM - 1) / kBM;
  const int tiles_n = narrow ? (N + kSBN - 1) / kSBN : (N + kBN - 1) / kBN;
  const int tiles = tiles_m * tiles_n;
  const bool deep = K / ksplit / kBK >= 12;  // long K loop: 3 stages, else 2 and a third workgroup
  const size_t smem = narrow ? (deep ? 3 : 2) * kStreamStageBytes : 2 * (size_t)(kBM + kBN) * kBK;
  if (ksplit < 1 || (ksplit > 1 && K % (ksplit * kBK) != 0))
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm: K does not split into whole 128-byte steps");
  if ((long)tiles_m * tiles_n * ksplit >= (1L << 24))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "int8 gemm: more than 2^24 output tiles");
  const bool full = vec_store && N % 16 == 0;  // no column tail: the lean instantiation
  const long cus = cu_count();
  if (M <= 64 && K % kBK == 0) {
    const int grid = ((N + 31) / 32) * ksplit;
    if constexpr (std::is_same<Epi, EpiI8>::value || std::is_same<Epi, EpiI32>::value) {
      // thousands of columns: fewer, longer workgroups (one round of the chip)
      if (ksplit == 1 && K % 256 == 0 && K <= 1024 && N >= 8192 && g_skinny16_enabled) {
        const int kw = K / 4;
#define LSH_WIDE(MB, NPAIR)                                                                    \
  launch<gemm_i8_skinny16_wide_kernel<Epi, MB, NPAIR>>((N + 32 * NPAIR - 1) / (32 * NPAIR), 256, 0, \
                                                       A, W, epi, M, N, K, kw, 0, vec_store, s)
        // 128 columns per workgroup while that is one round of the chip (32768 columns on 256
        // compute units), 256 beyond
        if (N <= 128 * cus) {
          if (M <= 16) return LSH_WIDE(1, 4);
          if (M <= 32) return LSH_WIDE(2, 4);
          return LSH_WIDE(4, 4);
        }
        if (M <= 16) return LSH_WIDE(1, 8);
        if (M <= 32) return LSH_WIDE(2, 8);
        return LSH_WIDE(4, 8);
#undef LSH_WIDE
      }
    }
    if ((K / ksplit) % 256 == 0 && g_skinny16_enabled) {
      // whole 64-byte slices for each of the four wavefronts: the 16 x 16 x 64 form
#define LSH_SKINNY16(MB, GZ)                                                                    \
  (full && (long)grid * 2 * (GZ) <= cus                                                          \
       ? launch<gemm_i8_skinny16_kernel<Epi, MB, true, 1>>(((N + 15) / 16), 256, 0, A, W, epi, M, \
                                                           N, K, K / ksplit / 4, 0, vec_store, s, \
                                                           ksplit, ksplit, GZ)                   \
   : full ? launch<gemm_i8_skinny16_kernel<Epi, MB, true>>(grid / ksplit, 256, 0, A, W, epi, M, N, \
                                                           K, K / ksplit / 4, 0, vec_store, s,    \
                                                           ksplit, ksplit, GZ)                    \
          : launch<gemm_i8_skinny16_kernel<Epi, MB, false>>(grid / ksplit, 256, 0, A, W, epi, M,  \
                                                            N, K, K / ksplit / 4, 0, vec_store,   \
                                                            s, ksplit, ksplit, GZ))
      // More than 16 rows: the 16-row blocks are dealt to as many workgroups per column block as
      // one round of the chip holds (measured: a wavefront with one block's fragments and
      // products in a row finishes sooner than one with two or four, and the weights read again
      // come from L2).
      const int blocks = (M + 15) / 16;  // 1 .. 4
      if (blocks == 1) return LSH_SKINNY16(1, 1);
      if (blocks == 2) {
        if ((long)grid * 2 <= cus) return LSH_SKINNY16(1, 2);
        return LSH_SKINNY16(2, 1);
      }
      if ((long)grid * blocks <= cus) {
        if (blocks == 3) return LSH_SKINNY16(1, 3);
        return LSH_SKINNY16(1, 4);
      }
      if ((long)grid * 2 <= cus) return LSH_SKINNY16(2, 2);
      return LSH_SKINNY16(4, 1);
#undef LSH_SKINNY16
    }
    if (M <= 32) {
      if (full)
        return launch<gemm_i8_skinny_kernel<Epi, 1, true>>(grid, 256, 0, A, W, epi, M, N, K, 0, 0,
                                                           vec_store, s, ksplit);
      return launch<gemm_i8_skinny_kernel<Epi, 1, false>>(grid, 256, 0, A, W, epi, M, N, K, 0, 0,
                                                          vec_store, s, ksplit);
    }
    if (full)
      return launch<gemm_i8_skinny_kernel<Epi, 2, true>>(grid, 256, 0, A, W, epi, M, N, K, 0, 0,
                                                         vec_store, s, ksplit);
    return launch<gemm_i8_skinny_kernel<Epi, 2, false>>(grid, 256, 0, A, W, epi, M, N, K, 0, 0,
                                                        vec_store, s, ksplit);
  }
  if constexpr (has_tile_kernel<Epi>::value) {
    if (stream && full && ksplit == 1 && g_tile_kernel_enabled) {
      const TileChoice c = choose_tile(M, N, K);
      const int tm = c.tm ? (M + c.tm - 1) / c.tm : 0, tn = c.tn ? (N + c.tn - 1) / c.tn : 0;
      switch (c.shape) {
        case kTile256x256:
          return launch<gemm_i8_tile_kernel<Epi, 2, 4, 4, 2, 2>>(tm * tn, 512, 2 * 512 * kBK, A, W,
                                                                 epi, M, N, K, tm, tn, true, s);
        case kTile256x192:
          return launch<gemm_i8_tile_kernel<Epi, 4, 2, 2, 3, 2>>(tm * tn, 512, 2 * 448 * kBK, A, W,
                                                                 epi, M, N, K, tm, tn, true, s);
        case kTile256x128:
          return launch<gemm_i8_tile_kernel<Epi, 4, 2, 2, 2, 3>>(tm * tn, 512, 3 * 384 * kBK, A, W,
                                                                 epi, M, N, K, tm, tn, true, s);
        case kTile128x96:
          // long K loops: a deeper ring (one workgroup per compute unit either way)
          if (K / kBK >= 12)
            return launch<gemm_i8_tile_kernel<Epi, 4, 1, 1, 3, 4>>(tm * tn, 256, 4 * 224 * kBK, A, W,
                                                                   epi, M, N, K, tm, tn, true, s);
          return launch<gemm_i8_tile_kernel<Epi, 4, 1, 1, 3, 2>>(tm * tn, 256, 2 * 224 * kBK, A, W,
                                                                 epi, M, N, K, tm, tn, true, s);
        default:
          break;
      }
    }
  }
  if constexpr (std::is_same<Epi, EpiLutI8>::value) {
    // the tabulated epilogue: 128 x 64 tiles, 2 stages + 16 KB of table rows in LDS
    if (stream && ksplit == 1 && K / kBK >= 2) {
      const int tn64 = (N + kSBN - 1) / kSBN;
      if ((long)tiles_m * tn64 >= (1L << 24))
        return lsh_fail(LSH_ERR_UNSUPPORTED, "int8 gemm: more than 2^24 output tiles");
      const int items = tiles_m * tn64;
      const size_t lds = 2 * kStreamStageBytes + (size_t)kSBN * 256;
      if (full)
        return launch<gemm_i8_stream_kernel<Epi, true, 2, true>>(items < 2 * cus ? items : (int)(2 * cus), 256, lds,
                                                                 A, W, epi, M, N, K, tiles_m, tn64,
                                                                 vec_store, s, 1);
      return launch<gemm_i8_stream_kernel<Epi, false, 2, true>>(items < 2 * cus ? items : (int)(2 * cus), 256, lds,
                                                                A, W, epi, M, N, K, tiles_m, tn64,
                                                                vec_store, s, 1);
    }
  }
  if (stream) {
    const int items = tiles * ksplit;
    // resident workgroups per compute unit: 2 (64 or 72 KB of LDS each) or 3 (48 KB)
    const int cap = (int)(narrow && !deep ? 3 * cus : 2 * cus);
    const int grid = items < cap ? items : cap;
    if (!narrow) {
      if (full)
        return launch<gemm_i8_stream128_kernel<Epi, true>>(grid, 256, smem, A, W, epi, M, N, K,
                                                           tiles_m, tiles_n, vec_store, s, ksplit);
      return launch<gemm_i8_stream128_kernel<Epi, false>>(grid, 256, smem, A, W, epi, M, N, K,
                                                          tiles_m, tiles_n, vec_store, s, ksplit);
    }
    if (deep) {
      if (full)
        return launch<gemm_i8_stream_kernel<Epi, true, 3>>(grid, 256, smem, A, W, epi, M, N, K,
                                                           tiles_m, tiles_n, vec_store, s, ksplit);
      return launch<gemm_i8_stream_kernel<Epi, false, 3>>(grid, 256, smem, A, W, epi, M, N, K,
                                                          tiles_m, tiles_n, vec_store, s, ksplit);
    }
    if (full)
      return launch<gemm_i8_stream_kernel<Epi, true, 2>>(grid, 256, smem, A, W, epi, M, N, K,
                                                         tiles_m, tiles_n, vec_store, s, ksplit);
    return launch<gemm_i8_stream_kernel<Epi, false, 2>>(grid, 256, smem, A, W, epi, M, N, K,
                                                        tiles_m, tiles_n, vec_store, s, ksplit);
  }
  if (ksplit != 1) return lsh_fail(LSH_ERR_UNSUPPORTED, "int8 gemm: this shape cannot split K");
  return launch<gemm_i8_generic_kernel<Epi>>(tiles, 256, smem, A, W, epi, M, N, K, tiles_m,
                                             tiles_n, vec_store, s);
}

bool gemm_i8_enable_tile_kernel(bool on) {
  const bool prev = g_tile_kernel_enabled.exchange(on);
  if (prev != on) route_epoch_bump();
  return prev;
}

bool gemm_i8_enable_skinny16_kernel(bool on) {
  const bool prev = g_skinny16_enabled.exchange(on);
  if (prev != on) route_epoch_bump();
  return prev;
}

std::string gemm_i8_kernel_name(int M, int N, int K, const char* epilogue) {
  if (M <= 64 && K % 256 == 0 && g_skinny16_enabled)
    return std::string("gemm_i8_skinny16_kernel<") + epilogue + ">";
  if (M <= 64 && K % kBK == 0) return std::string("gemm_i8_skinny_kernel<") + epilogue + ">";
  if (!stream_ok(M, N, K)) return std::string("gemm_i8_generic_kernel<") + epilogue + ">";
  const std::string e = epilogue ? epilogue : "";
  if (g_tile_kernel_enabled && N % 16 == 0 && choose_tile(M, N, K).shape != kTileNone) {
    return "gemm_i8_tile_kernel<" + e + ">";
  }
  if (e == "EpiLutI8" && K / kBK >= 2) return "gemm_i8_stream_kernel<EpiLutI8>";
  const bool wide = (e != "EpiI32" && e != "EpiI8") || !narrow_pays(M, N, K, 1);
  return std::string(wide ? "gemm_i8_stream128_kernel<" : "gemm_i8_stream_kernel<") + e + ">";
}

int gemm_i8_i32o(const int8_t* A, const int8_t* W, int32_t* C, int M, int N, int K,
                 hipStream_t s) {
  if (!C) return lsh_fail(LSH_ERR_INVALID, "int8 gemm: null output");
  return dispatch(A, W, EpiI32{C}, M, N, K, s);
}

// Heuristic split of K for int32-output products whose tile count leaves most of the 256
// compute units idle (N = hidden, K = inner size of the second FFN product).
int gemm_i8_preferred_ksplit(int M, int N, int K) {
  if (K % kBK != 0) return 1;
  const int nch = K / kBK;
  int items, per_item_min;
  if (M <= 64) {
    items = (N + 31) / 32;
    per_item_min = 4;  // one 128-byte step per wavefront
  } else {
    // at encoder sizes the int32 planes cost more HBM writes than the idle units cost time
    return 1;
  }
  int ks = 1;
  // (four planes: with one 16-column block per workgroup that is a round of the chip at hidden
  // 1024, and the layer norm that sums the planes has half as many to fetch as with eight --
  // measured over whole generation steps: 2 % (GPT-2-medium) and 3 % (Transformer-big) faster
  // than eight planes, two planes 3 % slower than four)
  while (ks < 4 && items * ks * 2 <= cu_count() && nch % (ks * 2) == 0 &&
         nch / (ks * 2) >= per_item_min)
    ks *= 2;
  return ks;
}

int gemm_i8_i32o_splitk(const int8_t* A, const int8_t* W, int32_t* C, int M, int N, int K,
                        int ksplit, int* used, hipStream_t s) {
  if (!C) return lsh_fail(LSH_ERR_INVALID, "int8 gemm: null output");
  if (ksplit < 1 || K % kBK != 0 || (K / kBK) % ksplit != 0 || (M > 64 && !stream_ok(M, N, K)))
    ksplit = 1;
  if (used) *used = ksplit;
  return dispatch(A, W, EpiI32{C}, M, N, K, s, ksplit);
}

int gemm_i8_i8o(const int8_t* A, const int8_t* W, int8_t* C, int M, int N, int K, float alpha,
                hipStream_t s) {
  if (!C) return lsh_fail(LSH_ERR_INVALID, "int8 gemm: null output");
  return dispatch(A, W, EpiI8{C, alpha}, M, N, K, s);
}

int gemm_i8_i8o_dev_alpha(const int8_t* A, const int8_t* W, int8_t* C, int M, int N, int K,
                          const float* alpha, hipStream_t s) {
  if (!C || !alpha) return lsh_fail(LSH_ERR_INVALID, "int8 gemm: null output or alpha");
  return dispatch(A, W, EpiI8Dev{C, alpha}, M, N, K, s);
}

int gemm_i8_bias_act_i8o(const int8_t* A, const int8_t* W, int8_t* C, const __half* bias, int M,
                         int N, int K, float alpha, float dequant_scale, float quant_scale,
                         float clip_max, int act, hipStream_t s) {
  if (!C || !bias) return lsh_fail(LSH_ERR_INVALID, "int8 gemm (bias+act): null pointer");
  switch (act) {
    case kActGelu:
      return dispatch(A, W, EpiActI8<kActGelu>{C, bias, alpha, dequant_scale, quant_scale, clip_max},
                      M, N, K, s);
    case kActRelu:
      return dispatch(A, W, EpiActI8<kActRelu>{C, bias, alpha, dequant_scale, quant_scale, clip_max},
                      M, N, K, s);
    case kActReluNarrow:
      return dispatch(A, W,
                      EpiActI8<kActReluNarrow>{C, bias, alpha, dequant_scale, quant_scale, clip_max},
                      M, N, K, s);
    default:
      return lsh_fail(LSH_ERR_INVALID, "int8 gemm (bias+act): unknown activation");
  }
}

int build_act_lut(int8_t* lut, const __half* bias, int N, float dequant_scale, float quant_scale,
                  float clip_max, int act, hipStream_t s) {
  if (!lut || !bias || N <= 0) return lsh_fail(LSH_ERR_INVALID, "build_act_lut: bad arguments");
  switch (act) {
    case kActGelu:
      build_act_lut_kernel<kActGelu><<<N, 256, 0, s>>>(lut, bias, N, dequant_scale, quant_scale,
                                                       clip_max);
      break;
    case kActRelu:
      build_act_lut_kernel<kActRelu><<<N, 256, 0, s>>>(lut, bias, N, dequant_scale, quant_scale,
                                                       clip_max);
      break;
    case kActReluNarrow:
      build_act_lut_kernel<kActReluNarrow><<<N, 256, 0, s>>>(lut, bias, N, dequant_scale,
                                                             quant_scale, clip_max);
      break;
    default:
      return lsh_fail(LSH_ERR_INVALID, "build_act_lut: unknown activation");
  }
  return lsh_check_launch("build_act_lut_kernel");
}

int gemm_i8_lut_i8o(const int8_t* A, const int8_t* W, int8_t* C, const int8_t* lut, int M, int N,
                    int K, float alpha, hipStream_t s) {
  if (!C || !lut) return lsh_fail(LSH_ERR_INVALID, "int8 gemm (table epilogue): null pointer");
  return dispatch(A, W, EpiLutI8{C, lut, alpha}, M, N, K, s);
}

int gemm_i8_decself_qkv_i8o(const int8_t* A, const int8_t* W, const __half* qkv_bias, int8_t* new_q,
                            int8_t* new_k, int8_t* new_v, int step_token_num, int hidden, int K,
                            int head_num, int max_step, int step_id, float alpha,
                            float dequant_scale, float quant_scale, hipStream_t s) {
  if (!qkv_bias || !new_q || !new_k || !new_v || head_num <= 0 || hidden <= 0 ||
      hidden % head_num != 0 || max_step <= 0)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm (decoder qkv): bad arguments");
  if (step_id < 0 || step_id >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm (decoder qkv): step_id outside the cache");
  const int d = hidden / head_num;
  if (d % 16 != 0 ||
      ((reinterpret_cast<uintptr_t>(qkv_bias) | reinterpret_cast<uintptr_t>(new_q) |
        reinterpret_cast<uintptr_t>(new_k) | reinterpret_cast<uintptr_t>(new_v)) & 15u) != 0)
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "int8 gemm (decoder qkv): needs dim_per_head % 16 == 0 and aligned outputs");
  if (step_token_num <= 64 && (long)step_token_num * hidden * max_step >= (1L << 31))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "int8 gemm (decoder qkv): a cache of 2^31 bytes or more at 64 rows or fewer");
  return dispatch(A, W,
                  EpiDecQkvI8{new_q, new_k, new_v, qkv_bias, alpha, dequant_scale, quant_scale,
                              hidden, head_num, d, max_step, step_id, 1.0f / (float)hidden,
                              1.0f / (float)d},
                  step_token_num, 3 * hidden, K, s);
}

int gemm_i8_encdec_q_f16(const int8_t* A, const int8_t* W, const __half* q_bias, __half* new_q,
                         int step_token_num, int hidden, int K, int beam_size, int head_num,
                         float alpha, float dequant_scale, hipStream_t s) {
  if (!q_bias || !new_q || head_num <= 0 || hidden <= 0 || hidden % head_num != 0 ||
      beam_size <= 0 || step_token_num <= 0 || step_token_num % beam_size != 0)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm (cross-attention q): bad arguments");
  const int d = hidden / head_num;
  if (d % 16 != 0 ||
      ((reinterpret_cast<uintptr_t>(q_bias) | reinterpret_cast<uintptr_t>(new_q)) & 15u) != 0)
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "int8 gemm (cross-attention q): needs dim_per_head % 16 == 0 and aligned output");
  return dispatch(A, W,
                  EpiEncdecQF16{new_q, q_bias, alpha, dequant_scale, beam_size, head_num, d,
                                1.0f / (float)beam_size, 1.0f / (float)d},
                  step_token_num, hidden, K, s);
}

int gemm_i8_qkv_arrange_f16(const int8_t* A, const int8_t* W, __half* new_qkv, const __half* qkv_bias,
                            long max_batch_dim, int batch_tokens, int hidden, int K, int seq_len,
                            int head_num, float alpha, float dequant_scale, hipStream_t s) {
  if (!new_qkv || !qkv_bias || seq_len <= 0 || head_num <= 0 || hidden % head_num != 0 ||
      batch_tokens % seq_len != 0 || max_batch_dim < (long)batch_tokens * hidden)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm (qkv arrange): bad arguments");
  const int d = hidden / head_num;
  if (d % 16 != 0 || max_batch_dim % 8 != 0 ||
      ((reinterpret_cast<uintptr_t>(new_qkv) | reinterpret_cast<uintptr_t>(qkv_bias)) & 15u) != 0)
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "int8 gemm (qkv arrange): needs dim_per_head % 16 == 0 and aligned output");
  return dispatch(A, W,
                  EpiQkvF16{new_qkv, qkv_bias, max_batch_dim, alpha, dequant_scale, seq_len,
                            head_num, d},
                  batch_tokens, 3 * hidden, K, s);
}

// Measurement aid: nothing but independent int8 MFMAs on register-resident operands, 8
// accumulator blocks per wavefront, 4 wavefronts per workgroup.  What the matrix units
// sustain at the clock the part holds under this load, as opposed to the nominal peak.
__global__ void __launch_bounds__(256)
mfma_i8_peak_kernel(int* __restrict__ out, int iters) {
  v4i a = {(int)threadIdx.x * 0x01010101, 0x7f81037d, 0x22e1c3a5, (int)blockIdx.x};
  v4i b = {0x5a3c1e7f, (int)threadIdx.x * 0x00010203, (int)0x81ff7f01u, 0x13579bdf};
  v16i c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) c[i] = (v16i)0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c[i], 0, 0, 0);
  }
  int sum = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) sum += c[i][j];
  out[blockIdx.x * 256 + threadIdx.x] = sum;
}

int mfma_i8_peak_probe(int* out, int workgroups, int iters, double* ops, hipStream_t s) {
  if (!out || workgroups <= 0 || iters <= 0)
    return lsh_fail(LSH_ERR_INVALID, "mfma_i8_peak_probe: bad arguments");
  mfma_i8_peak_kernel<<<workgroups, 256, 0, s>>>(out, iters);
  if (ops) *ops = (double)workgroups * 4 * iters * 8 * (2.0 * 32 * 32 * 32);
  return lsh_check_launch("mfma_i8_peak_kernel");
}

const char* gemm_i8_act_epilogue_name(int act) {
  return act == kActGelu ? EpiActI8<kActGelu>::name() : EpiActI8<kActRelu>::name();
}

}  // namespace lsh
