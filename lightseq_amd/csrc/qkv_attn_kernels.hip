// QKV projection and encoder self-attention of one (sequence, head) pair in one kernel.
//
// Replaces, for sequences of at most 128 tokens and heads of 64 dimensions, the chain
// inference/model/quant_bert_encoder.cc.cu:305-347 (int8 QKV GEMM -> ker_arrange_encself_qkv_i8I
// -> two strided batched GEMMs + ker_correlation_softmax_encself -> ker_arrange_atten_output_i8O):
// neither the int8 QKV codes [tokens, 3 * hidden] nor the fp16 q, k, v leave the compute unit.
//
// A workgroup (4 wavefronts) owns sequence b and head h:
//  1. the 128 x 192 int8 product X_b W_h^T (X_b: the tokens of the sequence, W_h: the 64 query,
//     64 key and 64 value rows of the head), K walked in 128-byte steps through a two-stage LDS
//     ring filled by global_load_lds_dwordx4, 64 x 96 accumulators per wavefront -- the loop of
//     the int8 GEMM tile kernel;
//  2. every accumulator becomes the int8 code the stand-alone GEMM would have stored
//     (requant_acc), then the fp16 value half(half(code * dq) + bias) that the arrange kernel
//     would have stored, and goes to LDS over the drained ring: queries and keys row-major,
//     values transposed;
//  3. the attention of one block of keys (attend_block128), context written as int8 codes.
// Results are byte-identical to the chain of stand-alone kernels.
#include "ls_device.h"
#include "ls_launch.h"
#include "tile_common.h"

#include <hip/hip_ext.h>

#include <atomic>
#include <mutex>
#include <type_traits>

namespace lsh {

namespace {
constexpr int kQaD = 64;                         // head size
constexpr int kQaTM = 128, kQaTN = 3 * kQaD;     // tokens x (q | k | v) columns of a workgroup
constexpr int kQaStage = (kQaTM + kQaTN) * kBK;  // bytes of one ring stage
constexpr int kQaNst = 2;
}  // namespace

// A plan (qkv_attention_plan) gives a workgroup its (sequence, head) pair and the number of
// 32-token blocks of the sequence that hold anything but padding.  Without one, workgroup w takes
// the pair of its index and the blocks up to the sequence length of the call.
constexpr int kQaItemHeadShift = 16, kQaItemBlocksShift = 28;

__global__ void __launch_bounds__(256, 2)
qkv_attn_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W,
                const _Float16* __restrict__ bias, const int* __restrict__ pad_mask,
                const int* __restrict__ plan, int8_t* __restrict__ ctx_q, float requant_alpha,
                float dq, float quant_scale, float alpha, int S, int batch, int head_num, int K) {
  constexpr int D = kQaD, WGN = 2, MB = 2, NB = 3, NWV = 4, TM = kQaTM, TN = kQaTN;
  constexpr int STAGE = kQaStage, NST = kQaNst;
  constexpr int NA = TM / 8 / NWV, NW = TN / 8 / NWV;  // 1-KB loads per wavefront
  extern __shared__ __align__(16) int8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN, l32 = lane & 31, g = lane >> 5;
  // Workgroups are dealt to the 8 XCDs round-robin; with a batch that is a multiple of 8 all
  // heads of a sequence run on one XCD, so its L2 fetches the sequence's activations once.
  int b, head, nblk;
  if (plan != nullptr) {
    const int item = __builtin_amdgcn_readfirstlane(plan[blockIdx.x]);
    b = item & 0xffff;
    head = (item >> kQaItemHeadShift) & 0xfff;
    nblk = (item >> kQaItemBlocksShift) & 7;
  } else {
    if ((batch & 7) == 0) {
      const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
      b = xcd + 8 * (j / head_num);
      head = j % head_num;
    } else {
      b = blockIdx.x / head_num;
      head = blockIdx.x % head_num;
    }
    nblk = (S + 31) >> 5;
  }
  const int hidden = head_num * D;
  const int nk = K / kBK;
  const int qi = wave * 32 + l32;  // the lane's query in the attention (wavefront w: block w)
  int8_t* out_row = ctx_q + ((long)b * S + qi) * hidden + head * D;
  if (nblk == 0) {
    // nothing but padding: the context of a padded query is zero
    if (qi < S) {
      uint4* o = reinterpret_cast<uint4*>(out_row + g * 32);
      o[0] = make_uint4(0, 0, 0, 0);
      o[1] = make_uint4(0, 0, 0, 0);
    }
    return;
  }

  // padding flags of keys `lane` and `64 + lane` (requested first, used after the product)
  const int pm0 = pad_mask[(long)b * S + min(lane, S - 1)];
  const int pm1 = pad_mask[(long)b * S + min(lane + 64, S - 1)];

  // Rows of the tile beyond block nblk are padding: they are not loaded, multiplied, converted
  // or attended.  Wavefront (wm, wn) owns the row blocks wm and wm + 2, so that the blocks that
  // exist spread over both wavefront rows.
  const bool live0 = wm < nblk, live1 = wm + 2 < nblk;
  uint32_t a_src[NA], w_src[NW];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int row = (wave + NWV * i) * 8 + (lane >> 3);  // row block i of the tile
    const int c = (lane & 7) ^ key_act(row);
    // tokens past the end of the sequence read its last token and are zeroed in step 2
    a_src[i] = (uint32_t)(b * S + min(row, S - 1)) * (uint32_t)K + c * 16;
  }
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int row = (wave + NWV * i) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ key_wgt(row);
    // tile column `row`: part row / 64 (q, k, v), dimension row % 64 of this head
    w_src[i] = (uint32_t)((row >> 6) * hidden + head * D + (row & 63)) * (uint32_t)K + c * 16;
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
  auto dma1 = [&](const int8_t* base, uint32_t voff, uint32_t lds) {
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff),
                 "s"(base)
                 : "memory");
  };
  auto issue = [&](int kt, int slot) {  // K step kt into ring slot `slot`
    const uint32_t base = lds0 + slot * STAGE;
#pragma unroll
    for (int i = 0; i < NA; ++i)
      if (i < nblk) dma1(A + kt * kBK, a_src[i], base + (wave + NWV * i) * 1024);
#pragma unroll
    for (int i = 0; i < NW; ++i)
      dma1(W + kt * kBK, w_src[i], base + TM * kBK + (wave + NWV * i) * 1024);
  };
  // LDS byte offset of this lane's fragment chunk for K slice 0; slice ks is at (offset ^ (ks << 5))
  int a_base[MB], w_base[NB];
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int row = (wm + 2 * i) * 32 + l32;
    a_base[i] = row * kBK + ((g ^ key_act(row)) << 4);
  }
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int row = wn * (NB * 32) + j * 32 + sigma(l32);
    w_base[j] = TM * kBK + row * kBK + ((g ^ key_wgt(row)) << 4);
  }
  struct Frag {
    v4i a[MB], w[NB];
  };
  v16i acc[MB][NB];

  // The product for a wavefront with LB of its two row blocks alive (2, 1 or 0: a wavefront
  // without rows still brings its share of the stages in and keeps the barriers).
  auto product = [&](auto lb_tag) {
    constexpr int LB = decltype(lb_tag)::value;
    auto load_frag = [&](Frag& f, const int8_t* stage, int ks) {
#pragma unroll
      for (int i = 0; i < LB; ++i)
        f.a[i] = *reinterpret_cast<const v4i*>(stage + (a_base[i] ^ (ks << 5)));
      if (LB > 0) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
          f.w[j] = *reinterpret_cast<const v4i*>(stage + (w_base[j] ^ (ks << 5)));
      }
    };
    // the first products of the tile start from a zero that is an operand of the instruction,
    // not cleared registers
    auto mma = [&](const Frag& f, auto first) {
#pragma unroll
      for (int i = 0; i < LB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
              f.w[j], f.a[i], decltype(first)::value ? (v16i)0 : acc[i][j], 0, 0, 0);
    };
    // issue order of one slice: an LDS read of the next slice after each of the first MFMAs
    auto pattern = [&]() {
      if (LB > 0) {
#pragma unroll
        for (int q = 0; q < LB + NB; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        if (LB * NB > LB + NB) __builtin_amdgcn_sched_group_barrier(0x008, LB * NB - (LB + NB), 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    Frag f[2];
    auto slices = [&](const int8_t* stage, auto first) {  // slices 1..3 read, slices 0..2 multiplied
#pragma unroll
      for (int ks = 1; ks < 4; ++ks) {
        load_frag(f[ks & 1], stage, ks);
        if (ks == 1) mma(f[0], first);
        else mma(f[(ks - 1) & 1], std::false_type{});
        pattern();
      }
    };
    static_assert(NST == 2, "the step below refills the slot it has just read");
    int slot = 0;
    // one K step but the last: multiply the stage in `slot`, then refill it with step kt + 2
    auto step = [&](int kt, auto first) {
      slices(smem + slot * STAGE, first);
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront has read all of the stage
      wait_vmcnt<0>();                     // its own loads of step kt + 1 have landed ...
      __builtin_amdgcn_s_barrier();        // ... and everyone's; everyone is done with step kt
      if (kt + NST < nk) issue(kt + NST, slot);
      __builtin_amdgcn_sched_barrier(0);
      slot ^= 1;
      load_frag(f[0], smem + slot * STAGE, 0);
      mma(f[1], std::false_type{});
      pattern();
    };
    load_frag(f[0], smem, 0);
    step(0, std::true_type{});
    for (int kt = 1; kt < nk - 1; ++kt) step(kt, std::false_type{});
    slices(smem + slot * STAGE, std::false_type{});
    mma(f[1], std::false_type{});
  };

#pragma unroll
  for (int s = 0; s < NST; ++s) issue(s, s);
  // the loads of stage 0 have landed once no more than stage 1's are outstanding: a wavefront
  // issues min(nblk, NA) + NW loads per stage
  if (nblk >= 4) wait_vmcnt<NA + NW>();
  else if (nblk == 3) wait_vmcnt<3 + NW>();
  else if (nblk == 2) wait_vmcnt<2 + NW>();
  else wait_vmcnt<1 + NW>();
  __builtin_amdgcn_s_barrier();
  if (live1) product(std::integral_constant<int, 2>{});
  else if (live0) product(std::integral_constant<int, 1>{});
  else product(std::integral_constant<int, 0>{});
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();  // the ring is drained: its memory now holds q, k, v

  // ---- step 2: accumulators -> int8 codes -> fp16 q, k (row-major) and v (transposed) ----
  constexpr int KSTR = attn_kstr(D), VSTR = kAttnVstr;
  _Float16* Qs = reinterpret_cast<_Float16*>(smem);
  _Float16* Ks = Qs + 128 * KSTR;
  _Float16* Vt = Ks + 128 * KSTR;
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    if (i == 0 ? !live0 : !live1) continue;
    const int t = (wm + 2 * i) * 32 + l32;  // token of the sequence
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      // this lane's 16 accumulators are columns wn * 96 + j * 32 + 16 g .. + 16 of the tile
      const int blk = wn * NB + j, part = blk >> 1, d0 = (blk & 1) * 32 + 16 * g;
      v8h lo, hi;
      requant_dequant16_bias(acc[i][j], requant_alpha, bias + part * hidden + head * D + d0, dq, lo,
                             hi);
      if (t >= S) lo = hi = (v8h)(_Float16)0;
      if (part == 2) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          Vt[(d0 + e) * VSTR + t] = lo[e];
          Vt[(d0 + 8 + e) * VSTR + t] = hi[e];
        }
      } else {
        _Float16* dst = (part == 0 ? Qs : Ks) + t * KSTR + d0;
        *reinterpret_cast<v8h*>(dst) = lo;
        *reinterpret_cast<v8h*>(dst + 8) = hi;
      }
    }
  }
  __syncthreads();

  // ---- step 3: attention; wavefront w owns queries 32 w .. 32 w + 31 ----
  if (wave >= nblk) {
    // queries that are all padding: zeros
    if (qi < S) {
      uint4* o = reinterpret_cast<uint4*>(out_row + g * 32);
      o[0] = make_uint4(0, 0, 0, 0);
      o[1] = make_uint4(0, 0, 0, 0);
    }
    return;
  }
  v8h qreg[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks)
    qreg[ks] = *reinterpret_cast<const v8h*>(&Qs[qi * KSTR + ks * 16 + g * 8]);
  const bool padk0 = pm0 != 0 || lane >= S, padk1 = pm1 != 0 || lane + 64 >= S;
  const uint64_t pad_q = __ballot(wave < 2 ? padk0 : padk1);
  const bool q_pad = qi >= S || ((pad_q >> ((wave & 1) * 32 + l32)) & 1) != 0;
  if (nblk >= 4)
    attend_block128<D, 4>(Ks, Vt, qreg, padk0, padk1, q_pad, qi < S, alpha, quant_scale, nullptr,
                          out_row, l32, g);
  else if (nblk == 3)
    attend_block128<D, 3>(Ks, Vt, qreg, padk0, padk1, q_pad, qi < S, alpha, quant_scale, nullptr,
                          out_row, l32, g);
  else if (nblk == 2)
    attend_block128<D, 2>(Ks, Vt, qreg, padk0, padk1, q_pad, qi < S, alpha, quant_scale, nullptr,
                          out_row, l32, g);
  else
    attend_block128<D, 1>(Ks, Vt, qreg, padk0, padk1, q_pad, qi < S, alpha, quant_scale, nullptr,
                          out_row, l32, g);
}

// ---------------------------------------------------------------------------------
// The plan of a launch: which (sequence, head) pair every workgroup takes and how many 32-token
// blocks of its sequence hold anything but padding.  The padding mask of an encoder call is
// the same for all its layers, so the plan is made once per call.
//
// Two workgroups fit a compute unit (80 KB of LDS each), and a launch of batch * heads of them
// is between one and two rounds of the chip: the compute units that hold two decide its length.
// Within an XCD (32 compute units; workgroup w runs on XCD w % 8, its position there is
// w / 8) the dispatcher gives positions 0..31 a compute unit each and position 32 + j the unit of
// position j.  So an XCD's pairs are listed longest sequence first for the positions up to 31
// and shortest first from 32 on: the longest meets the shortest.  The XCD's sequences are
// those whose rank by length is congruent to the XCD modulo 8 (all about equally long).
// ---------------------------------------------------------------------------------
constexpr int kQaPlanMaxBatch = 1024;

__global__ void __launch_bounds__(256)
qkv_attn_plan_kernel(const int* __restrict__ pad_mask, int* __restrict__ plan, int batch, int S,
                     int head_num) {
  __shared__ int len[kQaPlanMaxBatch];    // 1 + index of the last token that is not padding
  __shared__ int order[kQaPlanMaxBatch];  // order[rank] = sequence, longest first
  const int tid = threadIdx.x;
  for (int bb = tid; bb < batch; bb += 256) len[bb] = 0;
  __syncthreads();
  for (int i = tid; i < batch * S; i += 256)
    if (pad_mask[i] == 0) atomicMax(&len[i / S], i % S + 1);
  __syncthreads();
  for (int bb = tid; bb < batch; bb += 256) {
    int rank = 0;
    for (int o = 0; o < batch; ++o) rank += len[o] > len[bb] || (len[o] == len[bb] && o < bb);
    order[rank] = bb;
  }
  __syncthreads();
  const int items = batch * head_num;
  for (int w = tid; w < items; w += 256) {
    int seq_rank, head;
    if ((batch & 7) == 0) {
      const int xcd = w & 7, j = w >> 3, per_xcd = items >> 3;
      const int q = j < 32 ? j : per_xcd - 1 - (j - 32);  // list index: longest first
      seq_rank = xcd + 8 * (q / head_num);
      head = q % head_num;
    } else {
      seq_rank = w / head_num;
      head = w % head_num;
    }
    const int bb = order[seq_rank];
    plan[w] = bb | (head << kQaItemHeadShift) | (((len[bb] + 31) >> 5) << kQaItemBlocksShift);
  }
}

// The next launch on this thread records its begin / end timestamps into these events.
static thread_local hipEvent_t g_qa_ev_start = nullptr, g_qa_ev_stop = nullptr;
void qkv_attention_time_next_launch(hipEvent_t start, hipEvent_t stop) {
  g_qa_ev_start = start;
  g_qa_ev_stop = stop;
}

bool qkv_attention_fused_supported(int batch, int seq_len, int head_num, int dim_per_head) {
  const long hidden = (long)head_num * dim_per_head;
  return dim_per_head == kQaD && seq_len >= 1 && seq_len <= kQaTM && hidden % kBK == 0 &&
         hidden / kBK >= kQaNst && (long)batch * seq_len * hidden < (1l << 32) &&
         3 * hidden * hidden < (1l << 32);
}

// qkv_weight int8 [3 * hidden, hidden] (K-contiguous), qkv_bias fp16 [3 * hidden], x int8
// [batch * seq_len, hidden], pad_mask int32 [batch, seq_len] (non-zero = padding), ctx_q int8
// [batch * seq_len, hidden].  requant_alpha: int32 accumulator -> int8 QKV code (the alpha of the
// stand-alone requantising GEMM); dequant_scale: QKV code -> float; quant_scale: context -> int8.
static std::atomic<bool> g_qa_plan_enabled{true};
bool qkv_attention_plan_enable(bool on) {
  const bool prev = g_qa_plan_enabled.exchange(on);
  if (prev != on) route_epoch_bump();
  return prev;
}
bool qkv_attention_plan_enabled() { return g_qa_plan_enabled.load(std::memory_order_relaxed); }

bool qkv_attention_plan_supported(int batch, int seq_len, int head_num) {
  return batch >= 1 && batch <= kQaPlanMaxBatch && batch < (1 << kQaItemHeadShift) &&
         head_num >= 1 && head_num < (1 << (kQaItemBlocksShift - kQaItemHeadShift)) &&
         seq_len >= 1 && seq_len <= kQaTM;
}

// plan: batch * head_num ints, valid for launches with the same pad_mask, batch, seq_len and
// head_num
int qkv_attention_plan(const int* pad_mask, int* plan, int batch, int seq_len, int head_num,
                       hipStream_t s) {
  if (!pad_mask || !plan) return lsh_fail(LSH_ERR_INVALID, "qkv_attention_plan: null pointer");
  if (!qkv_attention_plan_supported(batch, seq_len, head_num))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "qkv_attention_plan: needs batch <= 1024, head_num < 4096, seq_len <= 128");
  qkv_attn_plan_kernel<<<1, 256, 0, s>>>(pad_mask, plan, batch, seq_len, head_num);
  return lsh_check_launch("qkv_attn_plan_kernel");
}

int qkv_attention_i8(const int8_t* x, const int8_t* qkv_weight, const __half* qkv_bias,
                     const int* pad_mask, int8_t* ctx_q, float requant_alpha, float dequant_scale,
                     float quant_scale, int batch, int seq_len, int head_num, int dim_per_head,
                     hipStream_t s, const int* plan) {
  if (!x || !qkv_weight || !qkv_bias || !pad_mask || !ctx_q || batch <= 0 || seq_len <= 0 ||
      head_num <= 0)
    return lsh_fail(LSH_ERR_INVALID, "qkv_attention_i8: bad arguments");
  if (!qkv_attention_fused_supported(batch, seq_len, head_num, dim_per_head))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "qkv_attention_i8: needs dim_per_head 64, seq_len <= 128, hidden % 128 == 0");
  if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qkv_weight) |
        reinterpret_cast<uintptr_t>(qkv_bias) | reinterpret_cast<uintptr_t>(ctx_q)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "qkv_attention_i8: pointers must be 16-byte aligned");
  constexpr size_t smem = (size_t)kQaNst * kQaStage;
  {
    // the ring is larger than the default dynamic LDS limit: raise it once per device
    static std::mutex mu;
    static unsigned long long raised = 0;
    int dev = 0;
    if (lsh_check_hip(hipGetDevice(&dev), "hipGetDevice")) return LSH_ERR_HIP;
    std::lock_guard<std::mutex> lock(mu);
    if (dev >= 64 || !((raised >> dev) & 1)) {
      if (lsh_check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_attn_kernel),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                        "hipFuncSetAttribute(qkv_attn_kernel)"))
        return LSH_ERR_HIP;
      if (dev < 64) raised |= 1ull << dev;
    }
  }
  const int hidden = head_num * dim_per_head;
  const float alpha = __half2float(__float2half_rn(sqrtf(1.f / (float)dim_per_head)));
  hipEvent_t e0 = g_qa_ev_start, e1 = g_qa_ev_stop;
  g_qa_ev_start = g_qa_ev_stop = nullptr;
  if (plan != nullptr && !qkv_attention_plan_supported(batch, seq_len, head_num))
    return lsh_fail(LSH_ERR_INVALID, "qkv_attention_i8: this shape has no plan");
  hipExtLaunchKernelGGL(qkv_attn_kernel, dim3(batch * head_num), dim3(256), smem, s, e0, e1, 0, x,
                        qkv_weight, reinterpret_cast<const _Float16*>(qkv_bias), pad_mask, plan,
                        ctx_q,
                        requant_alpha, dequant_scale, quant_scale, alpha, seq_len, batch, head_num,
                        hidden);
  return lsh_check_launch("qkv_attn_kernel");
}

}  // namespace lsh
