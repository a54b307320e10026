// Decode step: QKV projection of one head, cache append and self attention in one kernel.
//
// Replaces, for heads of 64 dimensions, the pair of launches
//   int8 QKV GEMM with ker_arrange_decself_qkv_i8I_i8O as its epilogue
//   (inference/model/quant_decoder.cc.cu:660-674, quant_gpt_encoder.cc.cu:640-653)
//   -> q.K, ker_fuse_softmax_new_value_i32I_i8O (quant_decoder.cc.cu:679-700)
// A decode step is bound by the latency of its launches, not by bytes: each launch removed is
// worth 4-6 us per layer.
//
// A workgroup of 8 wavefronts owns RG rows (beams) and one head:
//  1. the RG x 192 int8 product of the rows with the head's 64 query, 64 key and 64 value
//     weight rows: v_mfma_i32_16x16x64_i8 with the weights as the row operand, fragments
//     read straight from global memory (every weight byte is used once per workgroup), the
//     K range split over wavefront pairs and summed through LDS (integer sums: exact);
//  2. the epilogue of the stand-alone product (requant_acc -> dequant + bias -> cache code):
//     q to new_q, k and v to slot step_id of the caches -- the same bytes;
//  3. after a barrier (the rows just written are read back by the same workgroup), the
//     attention body of the stand-alone kernel (decself_attend_row), one group of NWV
//     wavefronts per row.
// With the group shape of the stand-alone kernel (NWV = 4) the context codes are the same
// bytes as the pair's; with one wavefront per row (short caches, many rows) the value sums
// run in another tree and a code can differ by one next to a rounding boundary.
#include "dec_attend.h"
#include "ls_device.h"
#include "ls_launch.h"

#include <atomic>

namespace lsh {

namespace {
std::atomic<bool> g_dqa_enabled{false};
constexpr int kDqaD = 64;          // head size
constexpr int kDqaCols = 3 * kDqaD;  // q | k | v columns of a head
typedef int dqa_v4i __attribute__((ext_vector_type(4)));
}  // namespace

template <int NWV, int UN, int RG>
__global__ void __launch_bounds__(512)
decself_qkv_attn_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ W,
                        const __half* __restrict__ bias, int8_t* new_q, int8_t* k_cache,
                        int8_t* v_cache, int8_t* __restrict__ ctx, int rows, int hidden,
                        int head_num, int max_step, int step_id, float alpha, float dequant_scale,
                        float cache_quant_scale, float attn_scale, float cache_dequant_scale,
                        float ctx_quant_scale) {
  static_assert(NWV * RG == 8, "8 wavefronts: RG groups of NWV");
  constexpr int D = kDqaD, COLS = kDqaCols;
  extern __shared__ float lds_f[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // workgroups are dealt to the 8 XCDs round-robin: with a head count that is a multiple of 8
  // a head's weights are fetched by one XCD's L2 only
  int head, rgp;
  if ((head_num & 7) == 0) {
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3, hp = head_num >> 3;
    head = xcd + 8 * (j % hp);
    rgp = j / hp;
  } else {
    head = blockIdx.x % head_num;
    rgp = blockIdx.x / head_num;
  }
  const int row0 = rgp * RG;
  const int step_num = step_id + 1;
  const long gfl = decself_group_floats<D, NWV>(step_num);
  int32_t* partial = reinterpret_cast<int32_t*>(lds_f + RG * gfl);  // [2][COLS][RG]

  // ---- 1. product: wavefront (kpart = wave & 1, blk0 = wave >> 1) owns K half kpart of the
  //         16-column blocks blk0, blk0 + 4, blk0 + 8 ----
  {
    const int kpart = wave & 1, blk0 = wave >> 1;
    const int KH = hidden >> 7;  // 64-byte K slices per half (<= 8)
    const int kq = lane >> 4;
    const int8_t* xp =
        x + (long)min(row0 + min(lane & 15, RG - 1), rows - 1) * hidden + (kpart * KH) * 64 + kq * 16;
    dqa_v4i xf[8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
      if (s < KH) xf[s] = *reinterpret_cast<const dqa_v4i*>(xp + s * 64);
    const int8_t* wp[3];
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      const int n = (blk0 + 4 * t) * 16 + (lane & 15);  // column of the head's q | k | v
      wp[t] = W + ((long)(n >> 6) * hidden + head * D + (n & 63)) * hidden + (kpart * KH) * 64 +
              kq * 16;
    }
    dqa_v4i wa[8], wb[8], acc[3];
    auto fetch = [&](dqa_v4i (&w)[8], int t) {
#pragma unroll
      for (int s = 0; s < 8; ++s)
        if (s < KH) w[s] = *reinterpret_cast<const dqa_v4i*>(wp[t] + s * 64);
    };
    auto mul = [&](const dqa_v4i (&w)[8], int t) {
      acc[t] = (dqa_v4i)0;
#pragma unroll
      for (int s = 0; s < 8; ++s)
        if (s < KH) acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[s], xf[s], acc[t], 0, 0, 0);
    };
    fetch(wa, 0);
    fetch(wb, 1);
    mul(wa, 0);
    fetch(wa, 2);
    mul(wb, 1);
    mul(wa, 2);
    // lane holds C[row lane % 16][block * 16 + 4 * (lane / 16) + 0..3]
    const int m = lane & 15;
    if (m < RG) {
#pragma unroll
      for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          partial[(kpart * COLS + (blk0 + 4 * t) * 16 + 4 * kq + i) * RG + m] = acc[t][i];
    }
  }
  __syncthreads();

  // ---- 2. epilogue of the stand-alone product: q, and slot step_id of the caches ----
  for (int idx = tid; idx < COLS * RG; idx += 512) {
#pragma clang fp contract(off)
    const int m = idx / COLS, n = idx - m * COLS;
    const int row = row0 + m;
    if (row >= rows) continue;
    const int sum = partial[n * RG + m] + partial[(COLS + n) * RG + m];
    const int part = n >> 6, dd = n & 63;
    const float b = __half2float(bias[(long)part * hidden + head * D + dd]);
    const float val = (float)requant_acc(sum, alpha) * dequant_scale + b;
    const int8_t code = (int8_t)float2int8(val, cache_quant_scale);
    if (part == 0) {
      new_q[(long)row * hidden + head * D + dd] = code;
    } else {
      int8_t* cache = part == 1 ? k_cache : v_cache;
      cache[(((long)row * head_num + head) * max_step + step_id) * D + dd] = code;
    }
  }
  __syncthreads();  // the group reads back what the workgroup has just written

  // ---- 3. attention: group g = row row0 + g ----
  {
    const int g = wave / NWV, wid = wave % NWV;
    const int row = min(row0 + g, rows - 1);
    const long bh = (long)row * head_num + head;
    decself_attend_row<D, NWV, UN>(new_q + bh * D, k_cache + bh * (long)max_step * D,
                                   v_cache + bh * (long)max_step * D,
                                   ctx + (long)row * hidden + head * D, row0 + g < rows, step_num,
                                   attn_scale, cache_dequant_scale, ctx_quant_scale,
                                   lds_f + g * gfl, wid, lane);
  }
}

// The same for caches of 257 to 1024 steps (one row and one head per workgroup, the eight
// wavefronts of the stand-alone attention over such a cache): the two streams of the pair --
// the head's weights and the row's cache -- are requested together at the start.  The cache
// rows do not depend on the projection except the one the step appends, so every lane loads
// its rows first (the appended row's slot holds old bytes), the product and its epilogue run
// while they travel, the epilogue leaves the new q, k and v codes in LDS as well as in memory,
// and the lane that owns the appended row takes it from there before it enters the attention
// body of the stand-alone kernel (decself_attend_row_once_body: the same bits).
template <int UN>
__global__ void __launch_bounds__(512)
decself_qkv_attn_early_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ W,
                              const __half* __restrict__ bias, int8_t* new_q, int8_t* k_cache,
                              int8_t* v_cache, int8_t* __restrict__ ctx, int rows, int hidden,
                              int head_num, int max_step, int step_id, float alpha,
                              float dequant_scale, float cache_quant_scale, float attn_scale,
                              float cache_dequant_scale, float ctx_quant_scale) {
  constexpr int D = kDqaD, COLS = kDqaCols, NWV = 8;
  constexpr int CH = D / 16, KPW = 64 / CH;
  extern __shared__ float lds_f[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int head, row;
  if ((head_num & 7) == 0) {
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3, hp = head_num >> 3;
    head = xcd + 8 * (j % hp);
    row = j / hp;
  } else {
    head = blockIdx.x % head_num;
    row = blockIdx.x / head_num;
  }
  const int step_num = step_id + 1;
  const long gfl = decself_group_floats<D, NWV>(step_num);
  int32_t* partial = reinterpret_cast<int32_t*>(lds_f + gfl);              // [2][COLS]
  int8_t* fresh = reinterpret_cast<int8_t*>(partial + 2 * COLS);           // q | k | v codes, [COLS]
  const long bh = (long)row * head_num + head;
  const int8_t* kb = k_cache + bh * (long)max_step * D;
  const int8_t* vb = v_cache + bh * (long)max_step * D;

  // ---- 0. the row's cache: requested before anything else ----
  uint4 kv[UN], vv[UN];
  decself_attend_load_rows<D, NWV, UN>(kb, vb, step_num, wave, lane, kv, vv);
  // (and the bias of the element this thread finishes in the epilogue)
  const __half bias_h = bias[(long)(min(tid, COLS - 1) >> 6) * hidden + head * D + (tid & 63)];

  // ---- 1. product: wavefront (kpart = wave & 1, blk0 = wave >> 1) owns K half kpart of the
  //         16-column blocks blk0, blk0 + 4, blk0 + 8 (matrix row 0 is the row) ----
  {
    const int kpart = wave & 1, blk0 = wave >> 1;
    const int KH = hidden >> 7;  // 64-byte K slices per half (<= 8)
    const int kq = lane >> 4;
    const int8_t* xp = x + (long)row * hidden + (kpart * KH) * 64 + kq * 16;
    dqa_v4i xf[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) xf[s] = *reinterpret_cast<const dqa_v4i*>(xp + min(s, KH - 1) * 64);
    const int8_t* wp[3];
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      const int n = (blk0 + 4 * t) * 16 + (lane & 15);  // column of the head's q | k | v
      wp[t] = W + ((long)(n >> 6) * hidden + head * D + (n & 63)) * hidden + (kpart * KH) * 64 +
              kq * 16;
    }
    dqa_v4i w[3][8], acc[3];
#pragma unroll
    for (int t = 0; t < 3; ++t)
#pragma unroll
      for (int s = 0; s < 8; ++s)
        w[t][s] = *reinterpret_cast<const dqa_v4i*>(wp[t] + min(s, KH - 1) * 64);
    __builtin_amdgcn_sched_barrier(0);  // every request of the kernel is out before a product
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      acc[t] = (dqa_v4i)0;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        asm volatile("" : "+v"(w[t][s]));
        if (t == 0) asm volatile("" : "+v"(xf[s]));
        if (s < KH) acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[t][s], xf[s], acc[t], 0, 0, 0);
      }
    }
    // lane holds C[row lane % 16][block * 16 + 4 * (lane / 16) + 0..3]; row 0 is the row
    if ((lane & 15) == 0) {
#pragma unroll
      for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          partial[kpart * COLS + (blk0 + 4 * t) * 16 + 4 * kq + i] = acc[t][i];
    }
  }
  __syncthreads();

  // ---- 2. epilogue of the stand-alone product, one element per thread: q to new_q, k and v
  //         to slot step_id of the caches, and all three to LDS ----
  if (tid < COLS) {
#pragma clang fp contract(off)
    const int n = tid;
    const int sum = partial[n] + partial[COLS + n];
    const int part = n >> 6, dd = n & 63;
    const float b = __half2float(bias_h);
    const float val = (float)requant_acc(sum, alpha) * dequant_scale + b;
    const int8_t code = (int8_t)float2int8(val, cache_quant_scale);
    fresh[n] = code;
    if (part == 0) {
      new_q[(long)row * hidden + head * D + dd] = code;
    } else {
      int8_t* cache = part == 1 ? k_cache : v_cache;
      cache[(bh * max_step + step_id) * D + dd] = code;
    }
  }
  __syncthreads();

  // ---- 3. attention: the lane that holds the appended row takes it from LDS ----
  {
    const int c = lane % CH, grp = lane / CH;
    const uint4 qv = *reinterpret_cast<const uint4*>(fresh + c * 16);
    const uint4 nk = *reinterpret_cast<const uint4*>(fresh + D + c * 16);
    const uint4 nv = *reinterpret_cast<const uint4*>(fresh + 2 * D + c * 16);
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int j = (u * NWV + wave) * KPW + grp;
      // rows beyond the cache were clamped to the appended one; they are masked in the body,
      // but take the new bytes all the same
      if (j >= step_id) {
        kv[u] = nk;
        vv[u] = nv;
      }
    }
    decself_attend_row_once_body<D, NWV, UN>(qv, kv, vv, ctx + (long)row * hidden + head * D,
                                             true, step_num, attn_scale, cache_dequant_scale,
                                             ctx_quant_scale, lds_f, wave, lane);
  }
}

bool decself_qkv_attention_enable(bool on) {
  const bool prev = g_dqa_enabled.exchange(on);
  if (prev != on) route_epoch_bump();
  return prev;
}
bool decself_qkv_attention_enabled() { return g_dqa_enabled.load(std::memory_order_relaxed); }

bool decself_qkv_attention_supported(int rows, int hidden, int head_num, int max_step) {
  return rows > 0 && head_num > 0 && hidden == head_num * kDqaD && hidden % 128 == 0 &&
         hidden <= 1024 && max_step > 0 && max_step <= 4096;
}

// x int8 [rows, hidden]; qkv_weight int8 [3 * hidden, hidden] (K-contiguous); qkv_bias fp16
// [3 * hidden]; new_q int8 [rows, hidden]; caches int8 [rows, heads, max_step, 64]; ctx int8
// [rows, hidden].  alpha, dequant_scale, cache_quant_scale: the three scales of
// gemm_i8_decself_qkv_i8o; attn_scale, cache_dequant_scale, ctx_quant_scale: those of
// decself_attention_i8 (step_num = step_id + 1).
int decself_qkv_attention_i8(const int8_t* x, const int8_t* qkv_weight, const __half* qkv_bias,
                             int8_t* new_q, int8_t* k_cache, int8_t* v_cache, int8_t* ctx,
                             int rows, int hidden, int head_num, int max_step, int step_id,
                             float alpha, float dequant_scale, float cache_quant_scale,
                             float attn_scale, float cache_dequant_scale, float ctx_quant_scale,
                             hipStream_t s) {
  if (!x || !qkv_weight || !qkv_bias || !new_q || !k_cache || !v_cache || !ctx)
    return lsh_fail(LSH_ERR_INVALID, "decself_qkv_attention_i8: null pointer");
  if (!decself_qkv_attention_supported(rows, hidden, head_num, max_step))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "decself_qkv_attention_i8: needs heads of 64, hidden % 128 == 0, hidden <= "
                    "1024, max_step <= 4096");
  if (step_id < 0 || step_id >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "decself_qkv_attention_i8: step_id outside the cache");
  if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qkv_weight) |
        reinterpret_cast<uintptr_t>(new_q) | reinterpret_cast<uintptr_t>(k_cache) |
        reinterpret_cast<uintptr_t>(v_cache)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "decself_qkv_attention_i8: pointers must be 16-byte aligned");
  const int step_num = step_id + 1;
  // Group shape by cache length only (a row's result must not depend on its batch): one
  // wavefront per row reads a short cache in one round; longer caches get four.
#define LSH_DQA(NWV, UN, RG)                                                                       \
  do {                                                                                             \
    const size_t lds = (size_t)(RG * decself_group_floats<kDqaD, NWV>(step_num)) * sizeof(float) + \
                       (size_t)2 * kDqaCols * RG * sizeof(int32_t);                                \
    const int grid = ((rows + RG - 1) / RG) * head_num;                                            \
    decself_qkv_attn_kernel<NWV, UN, RG><<<grid, 512, lds, s>>>(                                   \
        x, qkv_weight, qkv_bias, new_q, k_cache, v_cache, ctx, rows, hidden, head_num, max_step,   \
        step_id, alpha, dequant_scale, cache_quant_scale, attn_scale, cache_dequant_scale,         \
        ctx_quant_scale);                                                                          \
  } while (0)
#define LSH_DQA_EARLY(UN)                                                                          \
  do {                                                                                             \
    const size_t lds = (size_t)decself_group_floats<kDqaD, 8>(step_num) * sizeof(float) +          \
                       (size_t)2 * kDqaCols * sizeof(int32_t) + kDqaCols;                          \
    decself_qkv_attn_early_kernel<UN><<<rows * head_num, 512, lds, s>>>(                           \
        x, qkv_weight, qkv_bias, new_q, k_cache, v_cache, ctx, rows, hidden, head_num, max_step,   \
        step_id, alpha, dequant_scale, cache_quant_scale, attn_scale, cache_dequant_scale,         \
        ctx_quant_scale);                                                                          \
  } while (0)
  if (step_num <= 64) LSH_DQA(1, 4, 8);
  else if (step_num <= 128) LSH_DQA(4, 2, 2);
  else if (step_num <= 256) LSH_DQA(4, 4, 2);
  else if (step_num <= 1024) {
    // the group shape and loads per lane of the stand-alone attention at this length
    const int un8 = (step_num + 127) / 128;
    if (un8 <= 3) LSH_DQA_EARLY(3);
    else if (un8 == 4) LSH_DQA_EARLY(4);
    else if (un8 == 5) LSH_DQA_EARLY(5);
    else if (un8 == 6) LSH_DQA_EARLY(6);
    else LSH_DQA_EARLY(8);
  } else LSH_DQA(8, 8, 1);
#undef LSH_DQA_EARLY
#undef LSH_DQA
  return lsh_check_launch("decself_qkv_attn_kernel");
}

}  // namespace lsh
