// The feed-forward half of an encoder layer as ONE launch: FFN1 (int8 GEMM with the tabulated
// bias + activation + requantisation epilogue) -> FFN2 (int8 GEMM, int32 accumulators) ->
// dequantise + residual (+ column sums) + LayerNorm (+ quantise).  Replaces three launches of
// the layer loop (inference/model/quant_bert_encoder.cc.cu:414-520) and leaves the same bytes.
//
// Why one launch can do it: every step of the path is independent between token rows, so the
// rows are dealt to the 8 XCDs (rows_per_xcd consecutive rows each) and an XCD's 32 workgroups
// only ever wait for one another -- through the L2 they share, with no cache maintenance
// (xcd_sync.h).  The activation codes and the int32 accumulators of an XCD's rows are written
// to the usual buffers, but they are consumed out of that L2 before the launch ends; what the
// kernel boundaries of the three launches cost (first operands through a cold L2, write-back of
// 12.6 + 12.6 MB, two launch ramps) is not paid.
//
// Phases of a workgroup (512 threads, one workgroup per compute unit, grid = 8 * 32):
//   1. FFN1 tiles of 256 x 192 (tile_gemm on 8 wavefronts) of the XCD's rows, dealt round-robin;
//   -- XCD barrier --
//   2. FFN2 tiles of 128 x 96 (tile_gemm on wavefronts 0-3, 4-stage ring; wavefronts 4-7 only
//      keep the workgroup barriers), the activation operand read past the vector cache;
//   -- XCD barrier --
//   3. LayerNorm of groups of 16 (8) rows: the int32 rows come into LDS past the vector cache,
//      then the row routine of the stand-alone kernel runs on them.
// A wait that gives up (xcd_sync.h) ends the kernel; the host then sees the error word.
#include "ls_device.h"
#include "ls_launch.h"
#include "gemm_tile.h"
#include "ln_rows8.h"

#define LSH_XCD_FN __device__ __forceinline__
#include "xcd_sync.h"

#include <hip/hip_ext.h>

#include <atomic>
#include <mutex>

namespace lsh {

namespace {

struct XcdL2Mem {
  static __device__ __forceinline__ unsigned load(const unsigned* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void add(unsigned* p, unsigned v) {
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void fetch_or(unsigned* p, unsigned v) {
    __hip_atomic_fetch_or(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void pause() { __builtin_amdgcn_s_sleep(1); }
};

// XCC_ID (hardware register 20, bits 3:0): the XCD this wavefront runs on
__device__ __forceinline__ unsigned xcd_hw_id() {
  return __builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xf;
}

// Every wavefront of the workgroup calls it.  The workgroup's stores are in the L2 before it
// announces itself.  False: leave the kernel.
__device__ __forceinline__ bool xcd_barrier(unsigned* counter, unsigned target, unsigned* error,
                                            int spin_limit, int* s_go) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0)
    *s_go = xcd_arrive_and_wait<XcdL2Mem>(counter, target, error, spin_limit) ? 1 : 0;
  __syncthreads();
  return *s_go != 0;
}

constexpr int kSegThreads = 512;
constexpr int kSegSlots = 32;  // workgroups per XCD
constexpr size_t kSegLds = 2 * 448 * kBK;  // == 4 * 224 * kBK: both rings
static_assert(2 * 448 == 4 * 224, "the FFN1 and FFN2 rings use the same LDS");

}  // namespace

struct FfnSegmentArgs {
  const int8_t* x;        // [M, H] input codes of FFN1
  const int8_t* w1;       // [I, H]
  const int8_t* lut1;     // [I, 256]
  int8_t* act;            // [M, I] activation codes (FFN1 out, FFN2 in)
  const int8_t* w2;       // [H, I]
  int32_t* acc;           // [M, H] FFN2 accumulators
  __half* residual;       // [M, H] read; written unless `final_ln`
  __half* out_t;          // final_ln: [M, H] output (may alias residual)
  int8_t* out_q;          // !final_ln: [M, H] codes of the next layer's input
  const __half *scale, *bias, *residual_bias, *colsum;
  unsigned* counters;     // [8][kXcdCounterStride]
  unsigned* error;
  float alpha1, dequant_scale, quant_scale;
  int M, H, I, rows_per_xcd, is_post_ln, spin_limit;
  unsigned base;          // what the counters held before this launch
  unsigned launch;        // launches before this one
  unsigned long long* stamps;  // measurement aid: [256][8] 100 MHz clock values, or null
};

template <int LPR, int ITER, bool FINAL>
__global__ void __launch_bounds__(kSegThreads)
ffn_segment_kernel(const FfnSegmentArgs a) {
  extern __shared__ __align__(16) int8_t smem[];
  __shared__ int s_go;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // The dispatcher deals consecutive workgroups to consecutive XCDs, starting wherever the
  // previous kernel of the queue left off: the XCD is read from the hardware, and blockIdx / 8
  // numbers its workgroups.  That every (XCD, slot) pair is taken exactly once is checked: the
  // workgroup flips its bit of the XCD's mask (word 1 of the counter line, all bits equal
  // between launches) and must find it as the launch count says.
  const int xcd = (int)xcd_hw_id() & 7, slot = blockIdx.x >> 3;
  auto stamp = [&](int i) {
    if (a.stamps != nullptr && tid == 0) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      a.stamps[blockIdx.x * 8 + i] = __builtin_amdgcn_s_memrealtime();
    }
  };
  stamp(0);
  unsigned* counter = a.counters + xcd * kXcdCounterStride;
  bool slot_taken = false;
  if (tid == 0) {
    const unsigned old = __hip_atomic_fetch_xor(counter + 1, 1u << slot, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
    slot_taken = ((old >> slot) & 1u) != (a.launch & 1u);
  }
  const int row_lo = min(xcd * a.rows_per_xcd, a.M), row_hi = min(row_lo + a.rows_per_xcd, a.M);
  const int rows = row_hi - row_lo;

  // ---- phase 1: FFN1, 256 x 192 tiles ----
  {
    const EpiLutI8 epi{a.act, a.lut1, a.alpha1};
    const int tn1 = (a.I + 191) / 192, tiles = ((rows + 255) / 256) * tn1;
    for (int t = slot; t < tiles; t += kSegSlots) {
      const int p = t / tn1, cn = t - p * tn1;
      tile_gemm<EpiLutI8, 4, 2, 2, 3, 2, false>(a.x, a.w1, epi, row_lo + p * 256, row_hi, a.I, a.H,
                                                cn, smem);
      __syncthreads();  // the epilogue has read its table: the ring may be refilled
    }
  }
  if (slot_taken) XcdL2Mem::fetch_or(a.error, kXcdErrMapping);
  stamp(1);
  if (!xcd_barrier(counter, a.base + kSegSlots, a.error, a.spin_limit, &s_go)) return;
  stamp(2);

  // ---- phase 2: FFN2, 128 x 96 tiles on wavefronts 0-3 ----
  {
    const EpiI32 epi{a.acc};
    const int tn2 = (a.H + 95) / 96, tiles = ((rows + 127) / 128) * tn2;
    const int nk = a.I / kBK;
    for (int t = slot; t < tiles; t += kSegSlots) {
      const int p = t / tn2, cn = t - p * tn2;
      if (wave < 4) {
        tile_gemm<EpiI32, 4, 1, 1, 3, 4, true>(a.act, a.w2, epi, row_lo + p * 128, row_hi, a.H, a.I,
                                               cn, smem);
      } else {
        for (int i = 0; i < tile_gemm_barriers<EpiI32, 4>(nk); ++i) __builtin_amdgcn_s_barrier();
      }
      __syncthreads();
    }
  }
  stamp(3);
  if (!xcd_barrier(counter, a.base + 2 * kSegSlots, a.error, a.spin_limit, &s_go)) return;
  stamp(4);

  // ---- phase 3: LayerNorm, groups of RPI rows ----
  {
    constexpr int RPW = kWave / LPR, RPI = 8 * RPW;
    const int H = a.H;
    const int groups = (rows + RPI - 1) / RPI;
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    const long end_off = (long)row_hi * H * 4 - 16;  // last 16 bytes of the XCD's accumulator rows
    for (int gi = slot; gi < groups; gi += kSegSlots) {
      const int r0 = row_lo + gi * RPI;
      const int chunks = (RPI * H * 4 + 1023) / 1024;
      for (int c = wave; c < chunks; c += 8) {
        const long off = min((long)r0 * H * 4 + c * 1024 + lane * 16, end_off);
        const uint32_t lds = __builtin_amdgcn_readfirstlane(lds0 + c * 1024);
        // past the vector cache: other compute units of the XCD wrote these rows a moment ago
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 sc1" ::"s"(lds),
                     "v"((uint32_t)off), "s"(a.acc)
                     : "memory");
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      const int row = r0 + wave * RPW + lane / LPR;
      const int32_t* staged = reinterpret_cast<const int32_t*>(smem) - (long)r0 * H;
      if (FINAL) {
        ln_rows8_row<__half, int32_t, kLnResOut, LPR, ITER>(
            row, row < row_hi, lane % LPR, staged, a.residual, a.out_t, nullptr, a.scale, a.bias,
            nullptr, a.colsum, H, a.dequant_scale, 0.f, 0, 1, 0, nullptr, r0);
      } else {
        ln_rows8_row<__half, int32_t, kLnResQuant, LPR, ITER>(
            row, row < row_hi, lane % LPR, staged, a.residual, nullptr, a.out_q, a.scale, a.bias,
            a.residual_bias, a.colsum, H, a.dequant_scale, a.quant_scale, a.is_post_ln, 1, 0,
            nullptr, r0);
      }
      __syncthreads();
    }
  }
  stamp(5);
}

// ---------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------
static thread_local hipEvent_t g_seg_ev_start = nullptr, g_seg_ev_stop = nullptr;
void ffn_segment_time_next_launch(hipEvent_t start, hipEvent_t stop) {
  g_seg_ev_start = start;
  g_seg_ev_stop = stop;
}

// At most one holder of the segment kernel per process at a time: two launches of it that were
// each partly resident would wait for workgroups that the other one keeps off the compute units
// (both would give up after their poll limit; this keeps it from happening between the models
// of one process).
static std::atomic<const void*> g_segment_owner{nullptr};
static std::atomic<bool> g_segment_enabled{false};
bool ffn_segment_claim(const void* who) {
  const void* expected = nullptr;
  return g_segment_owner.compare_exchange_strong(expected, who) || expected == who;
}
void ffn_segment_release(const void* who) {
  const void* expected = who;
  g_segment_owner.compare_exchange_strong(expected, nullptr);
}
bool ffn_segment_enable(bool on) {
  const bool prev = g_segment_enabled.exchange(on);
  if (prev != on) route_epoch_bump();
  return prev;
}
bool ffn_segment_enabled() { return g_segment_enabled.load(std::memory_order_relaxed); }

// Measurement aid: device memory for 256 x 8 clock values (100 MHz) that the next launches fill
// per workgroup -- 0 start, 1 FFN1 done, 2 past the first barrier, 3 FFN2 done, 4 past the second
// barrier, 5 layer norm done; null switches it off.
static std::atomic<unsigned long long*> g_segment_stamps{nullptr};
void ffn_segment_stamps(unsigned long long* dev) { g_segment_stamps.store(dev); }

size_t ffn_segment_sync_words() { return (size_t)kXcdCount * kXcdCounterStride + 1; }

bool ffn_segment_supported(int M, int H, int I) {
  const long lim = 1l << 32;
  return M >= 8 && H % kBK == 0 && I % kBK == 0 && H / kBK >= 2 && I / kBK >= 4 && H % 16 == 0 &&
         I % 16 == 0 && H <= 1024 && H % 8 == 0 && (long)M * I < lim && (long)I * H < lim &&
         (long)M * H * 4 < lim && (long)I * 256 < lim;
}

namespace {

// one workgroup of the kernel per compute unit, all 256 of them resident at once
template <auto Kern>
int segment_ready(bool* ok) {
  static std::mutex mu;
  static int state[64] = {};  // per device: 0 unknown, 1 usable, 2 not usable
  int dev = 0;
  if (lsh_check_hip(hipGetDevice(&dev), "hipGetDevice")) return LSH_ERR_HIP;
  std::lock_guard<std::mutex> lock(mu);
  if (dev < 64 && state[dev] != 0) {
    *ok = state[dev] == 1;
    return LSH_OK;
  }
  if (lsh_check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(Kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSegLds),
                    "hipFuncSetAttribute(ffn_segment_kernel)"))
    return LSH_ERR_HIP;
  int per_cu = 0, cus = 0;
  if (lsh_check_hip(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, Kern, kSegThreads, kSegLds),
                    "hipOccupancyMaxActiveBlocksPerMultiprocessor"))
    return LSH_ERR_HIP;
  if (lsh_check_hip(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev),
                    "hipDeviceGetAttribute"))
    return LSH_ERR_HIP;
  *ok = per_cu >= 1 && cus == kXcdCount * kSegSlots;
  if (dev < 64) state[dev] = *ok ? 1 : 2;
  return LSH_OK;
}

template <int LPR, int ITER, bool FINAL>
int launch_segment(const FfnSegmentArgs& a, hipStream_t s) {
  bool ok = false;
  if (int rc = segment_ready<ffn_segment_kernel<LPR, ITER, FINAL>>(&ok)) return rc;
  if (!ok)
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "ffn_segment: needs 256 compute units that each hold one workgroup of the kernel");
  hipEvent_t e0 = g_seg_ev_start, e1 = g_seg_ev_stop;
  g_seg_ev_start = g_seg_ev_stop = nullptr;
  hipExtLaunchKernelGGL((ffn_segment_kernel<LPR, ITER, FINAL>), dim3(kXcdCount * kSegSlots),
                        dim3(kSegThreads), kSegLds, s, e0, e1, 0, a);
  return lsh_check_launch("ffn_segment_kernel");
}

}  // namespace

// x int8 [M, H] -> act = lut1[FFN1(x)] int8 [M, I] -> acc = FFN2(act) int32 [M, H] -> layer
// norm of acc * dequant_scale + residual (+ colsum).  final_ln: fp16 out_t (may alias
// residual), residual only read; otherwise int8 out_q and the residual stream updated in
// place (residual_bias pre-added), as ker_residual_bias_ln_i32I_i8O.  sync: ffn_segment_sync_words()
// unsigned words of device memory, zero before the first launch; *launches: how many launches
// have used `sync` (the host's count of the barrier rounds, advanced here).  After a launch whose
// error word (sync[words - 1]) is non-zero the results are undefined and `sync` and *launches
// must be cleared before the next one.
int ffn_segment_i8(const int8_t* x, const int8_t* w1, const int8_t* lut1, float alpha1, int8_t* act,
                   const int8_t* w2, int32_t* acc, __half* residual, __half* out_t, int8_t* out_q,
                   const __half* scale, const __half* bias, const __half* residual_bias,
                   const __half* colsum, int M, int H, int I, float dequant_scale,
                   float quant_scale, bool is_post_ln, bool final_ln, unsigned* sync,
                   unsigned* launches, int spin_limit, hipStream_t s) {
  if (!x || !w1 || !lut1 || !act || !w2 || !acc || !residual || !scale || !bias || !sync ||
      !launches || (final_ln ? !out_t : !out_q) || spin_limit <= 0)
    return lsh_fail(LSH_ERR_INVALID, "ffn_segment: bad arguments");
  if (!ffn_segment_supported(M, H, I))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "ffn_segment: shape not covered");
  const uintptr_t align = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w1) |
                          reinterpret_cast<uintptr_t>(lut1) | reinterpret_cast<uintptr_t>(act) |
                          reinterpret_cast<uintptr_t>(w2) | reinterpret_cast<uintptr_t>(acc) |
                          reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(out_t) |
                          reinterpret_cast<uintptr_t>(out_q) | reinterpret_cast<uintptr_t>(scale) |
                          reinterpret_cast<uintptr_t>(bias) |
                          reinterpret_cast<uintptr_t>(residual_bias) |
                          reinterpret_cast<uintptr_t>(colsum);
  if (align & 15u) return lsh_fail(LSH_ERR_INVALID, "ffn_segment: pointers must be 16-byte aligned");
  FfnSegmentArgs a;
  a.x = x; a.w1 = w1; a.lut1 = lut1; a.act = act; a.w2 = w2; a.acc = acc;
  a.residual = residual; a.out_t = out_t; a.out_q = out_q;
  a.scale = scale; a.bias = bias; a.residual_bias = residual_bias; a.colsum = colsum;
  a.counters = sync;
  a.error = sync + kXcdCount * kXcdCounterStride;
  a.alpha1 = alpha1; a.dequant_scale = dequant_scale; a.quant_scale = quant_scale;
  a.M = M; a.H = H; a.I = I;
  // rows of an XCD: an eighth of the rows, in whole groups of 16 (a layer-norm pass)
  a.rows_per_xcd = ((M + 7) / 8 + 15) / 16 * 16;
  a.is_post_ln = is_post_ln ? 1 : 0;
  a.spin_limit = spin_limit;
  a.base = *launches * 2u * kSegSlots;
  a.launch = *launches;
  a.stamps = g_segment_stamps.load();
  *launches += 1;
#define LSH_SEG(LPR, IT) \
  (final_ln ? launch_segment<LPR, IT, true>(a, s) : launch_segment<LPR, IT, false>(a, s))
  if (H <= 256) return LSH_SEG(32, 1);
  if (H <= 512) return LSH_SEG(32, 2);
  if (H <= 768) return LSH_SEG(32, 3);
  return LSH_SEG(64, 2);
#undef LSH_SEG
}

}  // namespace lsh
