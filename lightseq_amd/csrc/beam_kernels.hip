// Beam search over int8 logits.
//
// Two families live here.
//  * The kernels behind the launchers of the reference, with their buffers and
//    meaning: candidate selection with the "rough top-k" threshold, the result and
//    cache refresh that consume globally sorted candidates, and the output writers.
//    The candidate set is exactly the reference's; candidates are emitted row by row
//    in ascending vocabulary order instead of in an order decided by atomics.
//  * The search step the decoder itself runs: an exact per-row top-k followed by a
//    per-sentence merge that also refreshes the sequences and scores.  It selects
//    the same beams as sorting the reference's candidates (any candidate among a
//    sentence's best `beam_size` is among its row's best `beam_size`, and the rough
//    threshold never cuts into a row's best `beam_size`), without a global sort, a
//    prefix scan or a device-to-host round trip.  Ties go to the lower candidate id.
#include "ls_device.h"

#include <type_traits>
#include "ls_launch.h"

#include <mutex>

namespace lsh {

constexpr float kMinLogProb = -2000.f;      // inference/kernels/transformerKernels.h:12
constexpr float kLogitThreshMin = -64.f;    // inference/kernels/transformerKernels.h:11
constexpr float kSeqLenEpsilon = 1e-12f;    // inference/kernels/transformerKernels.h:13

template <typename T>
__device__ __forceinline__ float logit_of(const int8_t* __restrict__ lr,
                                          const T* __restrict__ bias, int v, float dq) {
#pragma clang fp contract(off)
  return (float)lr[v] * dq + TT<T>::ld(bias, v);
}

__device__ __forceinline__ float cand_score(float lgt, float base, float length_norm,
                                            int batch_id) {
#pragma clang fp contract(off)
  return fmaxf((lgt + base) * length_norm, kMinLogProb + 1.f) + (float)batch_id * kMinLogProb;
}

// Row statistics shared by every selection kernel: max logit, sum of exp and (when
// `threads` > 0) the rough top-k threshold of inference/kernels/common.h:118-137 as a
// block of `threads` threads would compute it -- thread t of that block sees the
// vocabulary ids congruent to t modulo `threads`; `threads` is a power of two <= 1024
// so a lane of this 1024-thread block always stays inside one such class.
struct RowStats {
  float max_logit, sum_exp, topk;
};

// integer block sum for blocks of up to 1024 threads; `red` holds >= 16 ints
__device__ __forceinline__ int block_sum_i(int v, int* red) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, 64);
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  int r = 0;
  for (int i = 0; i < nw; ++i) r += red[i];
  return r;
}

template <typename T>
__device__ RowStats row_stats(const int8_t* __restrict__ lr, const T* __restrict__ bias,
                              int vocab, float dq, int threads, int K, float* red /*[1024+32]*/) {
  const int t = threadIdx.x;
  float tmax = kFloatInfNeg;
  for (int v = t; v < vocab; v += 1024) tmax = fmaxf(tmax, logit_of(lr, bias, v, dq));
  RowStats st;
  st.max_logit = block_max(tmax, red);
  float se = 0.f;
  for (int v = t; v < vocab; v += 1024)
    se += __expf(fmaxf(logit_of(lr, bias, v, dq) - st.max_logit, kLogitThreshMin));
  st.sum_exp = block_sum(se, red);
  st.topk = 0.f;
  if (threads > 0) {
    float* tm = red + 32;
    __syncthreads();
    tm[t] = tmax;
    __syncthreads();
    if (t < 32) {  // maximum of warp t of the emulated block
      float g = 0.f;
      if (t < (threads >> 5)) {
        g = kFloatInfNeg;
        for (int u = 0; u < 1024; ++u)
          if (((u & (threads - 1)) >> 5) == t) g = fmaxf(g, tm[u]);
      }
      red[t] = g;
    }
    __syncthreads();
    float best = 0.f;
    for (int r = 0; r < K; ++r) {
      float m = red[r];
      for (int j = r + K; j < 32; j += K) m = fmaxf(m, red[j]);
      best = r == 0 ? m : fminf(best, m);
    }
    st.topk = best;
    __syncthreads();
  }
  return st;
}

// ---------------------------------------------------------------------------------
// select_beam_rough_topk_i8I (inference/kernels/transformerKernels_int8.cc.cu:1690-1890)
// pass 1: candidates per row -> num_beam_can[1 + row]
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(1024)
beam_select_count_kernel(const int8_t* __restrict__ logits, const T* __restrict__ logit_bias,
                         const int* __restrict__ alive_seq, float dq, int* __restrict__ num_beam_can,
                         int vocab, int max_step, int cur_step, int threads, int beam_size,
                         int end_id) {
  __shared__ float red[1024 + 32];
  const int row = blockIdx.x;
  if (cur_step != 0 && alive_seq[(long)row * max_step + cur_step] == end_id) {
    if (threadIdx.x == 0) num_beam_can[row + 1] = 1;
    return;
  }
  const int8_t* lr = logits + (long)row * vocab;
  const RowStats st = row_stats(lr, logit_bias, vocab, dq, threads, beam_size, red);
  int n = 0;
  for (int v = threadIdx.x; v < vocab; v += 1024)
    n += logit_of(lr, logit_bias, v, dq) >= st.topk ? 1 : 0;
  n = block_sum_i(n, reinterpret_cast<int*>(red));
  if (threadIdx.x == 0) num_beam_can[row + 1] = n;
}

// pass 2: emit at the row's offset (sum of the preceding counts), ascending vocab id
template <typename T>
__global__ void __launch_bounds__(1024)
beam_select_emit_kernel(const int8_t* __restrict__ logits, const T* __restrict__ logit_bias,
                        const float* __restrict__ seq_probs, const float* __restrict__ seq_score,
                        const int* __restrict__ alive_seq, float dq, int* __restrict__ can_idx,
                        float* __restrict__ can_score, int* __restrict__ num_beam_can, int vocab,
                        int max_step, float length_norm, int cur_step, int rows, int threads,
                        int beam_size, int end_id) {
#pragma clang fp contract(off)
  __shared__ float red[1024 + 32];
  __shared__ int wave_cnt[16];
  __shared__ int s_base;
  const int row = blockIdx.x, t = threadIdx.x;
  const int lane = t & 63, wid = t >> 6;
  // offset of this row = candidates of the rows before it
  int ahead = 0, all = 0;
  for (int r = t; r < rows; r += 1024) {
    const int c = num_beam_can[r + 1];
    all += c;
    if (r < row) ahead += c;
  }
  const int pos = block_sum_i(ahead, reinterpret_cast<int*>(red));
  if (row == 0) {
    all = block_sum_i(all, reinterpret_cast<int*>(red));
    if (t == 0) num_beam_can[0] = all;
  }
  const int batch_id = row / beam_size;
  if (cur_step != 0 && alive_seq[(long)row * max_step + cur_step] == end_id) {
    if (t == 0) {  // a finished beam keeps its score and proposes <eos> once
      can_score[pos] = seq_score[row];
      can_idx[pos] = end_id + (row % beam_size) * vocab;
    }
    return;
  }
  const int8_t* lr = logits + (long)row * vocab;
  const RowStats st = row_stats(lr, logit_bias, vocab, dq, threads, beam_size, red);
  const float base = seq_probs[row] - logf(st.sum_exp) - st.max_logit;
  if (t == 0) s_base = pos;
  __syncthreads();
  for (int v0 = 0; v0 < vocab; v0 += 1024) {
    const int v = v0 + t;
    float lgt = 0.f;
    bool take = false;
    if (v < vocab) {
      lgt = logit_of(lr, logit_bias, v, dq);
      take = lgt >= st.topk;
    }
    const unsigned long long ballot = __ballot(take);
    if (lane == 0) wave_cnt[wid] = __popcll(ballot);
    __syncthreads();
    int off = s_base;
    for (int w2 = 0; w2 < wid; ++w2) off += wave_cnt[w2];
    off += __popcll(ballot & ((1ull << lane) - 1ull));
    if (take) {
      can_score[off] = cand_score(lgt, base, length_norm, batch_id);
      can_idx[off] = (row - batch_id * beam_size) * vocab + v;
    }
    __syncthreads();
    if (t == 0) {
      int tot = 0;
      for (int w2 = 0; w2 < 16; ++w2) tot += wave_cnt[w2];
      s_base += tot;
    }
    __syncthreads();
  }
}

template <typename T>
int select_beam_rough_topk_i8I(const int8_t* logits, const T* logit_bias, const float* seq_probs,
                               const float* seq_score, const int* alive_seq, float dequant_scale,
                               int* can_idx, float* can_score, int* num_beam_can, int vocab_size,
                               int max_step, float length_norm, int cur_step, int step_token_num,
                               int max_thread_per_block, hipStream_t s, int beam_size,
                               float diverse_lambda, int end_id) {
  if (!logits || !logit_bias || !seq_probs || !seq_score || !alive_seq || !can_idx ||
      !can_score || !num_beam_can || vocab_size <= 0 || step_token_num <= 0 || max_step <= 0 ||
      cur_step < 0 || cur_step >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "select_beam_rough_topk_i8I: bad arguments");
  if (diverse_lambda != 0.f)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "select_beam_rough_topk_i8I: diverse beam search");
  if (beam_size < 1 || beam_size > 32 || (beam_size & (beam_size - 1)) ||
      step_token_num % beam_size != 0)
    return lsh_fail(LSH_ERR_INVALID, "wrong beam_size, should be 1, 2, 4, 8, 16 or 32");
  const int th = max_thread_per_block;
  if (th < 32 || th > 1024 || (th & (th - 1)))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "select_beam_rough_topk_i8I: max_thread_per_block must be a power of two in "
                    "[32, 1024]");
  beam_select_count_kernel<T><<<step_token_num, 1024, 0, s>>>(
      logits, logit_bias, alive_seq, dequant_scale, num_beam_can, vocab_size, max_step, cur_step,
      th, beam_size, end_id);
  if (int rc = lsh_check_launch("beam_select_count_kernel")) return rc;
  beam_select_emit_kernel<T><<<step_token_num, 1024, 0, s>>>(
      logits, logit_bias, seq_probs, seq_score, alive_seq, dequant_scale, can_idx, can_score,
      num_beam_can, vocab_size, max_step, length_norm, cur_step, step_token_num, th, beam_size,
      end_id);
  return lsh_check_launch("beam_select_emit_kernel");
}
template int select_beam_rough_topk_i8I<float>(const int8_t*, const float*, const float*,
                                               const float*, const int*, float, int*, float*, int*,
                                               int, int, float, int, int, int, hipStream_t, int,
                                               float, int);
template int select_beam_rough_topk_i8I<__half>(const int8_t*, const __half*, const float*,
                                                const float*, const int*, float, int*, float*,
                                                int*, int, int, float, int, int, int, hipStream_t,
                                                int, float, int);

// ---------------------------------------------------------------------------------
// ker_refresh_result (inference/kernels/transformerKernels.cc.cu:1398-1463),
// diverse_lambda == 0.  Grid (batch, beam), one thread per position.
// ---------------------------------------------------------------------------------
__global__ void refresh_result_kernel(const int* __restrict__ can_idx,
                                      const float* __restrict__ can_score,
                                      const int* __restrict__ num_can_per_beam,
                                      const int* __restrict__ old_alive_seq,
                                      int* __restrict__ new_alive_seq, float* seq_probs,
                                      float* seq_score, int* num_finish_beam, int vocab_size,
                                      int cur_step, float length_norm, int end_id, int max_step) {
#pragma clang fp contract(off)
  const int b = blockIdx.x, j = blockIdx.y, beam = gridDim.y;
  const int can_pos = num_can_per_beam[b * beam] + j;
  const int ori = can_idx[can_pos];
  const int can_beam_id = ori / vocab_size, can_vocab_id = ori % vocab_size;
  for (int t = threadIdx.x; t < max_step; t += blockDim.x) {
    int tok;
    if (t > cur_step + 1)
      tok = end_id;
    else if (t == cur_step + 1)
      tok = can_vocab_id;
    else
      tok = old_alive_seq[((long)b * beam + can_beam_id) * max_step + t];
    new_alive_seq[((long)b * beam + j) * max_step + t] = tok;
  }
  if (threadIdx.x == 0) {
    if (can_vocab_id != end_id) {
      seq_probs[b * beam + j] = (can_score[can_pos] - (float)b * kMinLogProb) / length_norm;
    } else {
      atomicAdd(num_finish_beam, 1);
      seq_score[b * beam + j] = can_score[can_pos];
    }
  }
}

int refresh_result(const int* can_idx, const float* can_score, const int* num_can_per_beam,
                   const int* old_alive_seq, int* new_alive_seq, float* seq_probs,
                   float* seq_score, int* num_finish_beam, int vocab_size, int cur_step,
                   float length_norm, float diverse_lambda, int end_id, int batch_size,
                   int beam_size, int max_step, hipStream_t s) {
  if (!can_idx || !can_score || !num_can_per_beam || !old_alive_seq || !new_alive_seq ||
      !seq_probs || !seq_score || !num_finish_beam || batch_size <= 0 || beam_size <= 0 ||
      vocab_size <= 0 || max_step <= 0 || cur_step < 0 || cur_step + 1 >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "ker_refresh_result: bad arguments");
  if (diverse_lambda != 0.f)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "ker_refresh_result: diverse beam search");
  if (old_alive_seq == new_alive_seq)
    return lsh_fail(LSH_ERR_INVALID, "ker_refresh_result: the sequence buffers must differ");
  refresh_result_kernel<<<dim3(batch_size, beam_size), 256, 0, s>>>(
      can_idx, can_score, num_can_per_beam, old_alive_seq, new_alive_seq, seq_probs, seq_score,
      num_finish_beam, vocab_size, cur_step, length_norm, end_id, max_step);
  return lsh_check_launch("refresh_result_kernel");
}

// ---------------------------------------------------------------------------------
// K/V cache reorder after a search step
// (inference/kernels/transformerKernels.cc.cu:1579-1627 and its launcher :1657-1681).
// Grid (layer, 2 * rows).  The parent beam comes either from the sorted candidates
// (reference launcher) or from a parent table (-1 = finished beam, nothing copied).
// ---------------------------------------------------------------------------------
template <bool PARENT_TABLE>
__global__ void __launch_bounds__(256)
refresh_cache_kernel(const int* __restrict__ num_can_per_beam, const int* __restrict__ can_idx,
                     const int* __restrict__ parent, const int8_t* __restrict__ k_old,
                     const int8_t* __restrict__ v_old, int8_t* __restrict__ k_new,
                     int8_t* __restrict__ v_new, long layer_offset, int beam_size, int d,
                     int head_num, int vocab_size, int cur_step, int max_step, int end_id) {
  const int layer = blockIdx.x, kv = blockIdx.y & 1, row = blockIdx.y >> 1;
  const int b = row / beam_size, j = row % beam_size;
  int src;
  if (PARENT_TABLE) {
    src = parent[row];
    if (src < 0) return;
  } else {
    const int c = can_idx[num_can_per_beam[b * beam_size] + j];
    if (c % vocab_size == end_id) return;
    src = c / vocab_size;
  }
  if (src < 0 || src >= beam_size) return;  // never read outside the sentence's beams
  const long beam_bytes = (long)head_num * max_step * d;
  const long o = layer * layer_offset + ((long)b * beam_size + src) * beam_bytes;
  const long n = layer * layer_offset + ((long)b * beam_size + j) * beam_bytes;
  const int8_t* from = (kv ? v_old : k_old) + o;
  int8_t* to = (kv ? v_new : k_new) + n;
  const int chunk = (cur_step + 1) * d;  // contiguous bytes per head
  const long head_stride = (long)max_step * d;
  const bool vec = (d % 16 == 0) && (layer_offset % 16 == 0) &&
                   ((reinterpret_cast<uintptr_t>(from) | reinterpret_cast<uintptr_t>(to)) & 15u) == 0;
  if (vec) {
    const int per_head = chunk >> 4;
    for (int i = threadIdx.x; i < per_head * head_num; i += blockDim.x) {
      const int h = i / per_head, c16 = i % per_head;
      const long p = h * head_stride + (long)c16 * 16;
      *reinterpret_cast<uint4*>(to + p) = *reinterpret_cast<const uint4*>(from + p);
    }
  } else {
    for (int i = threadIdx.x; i < chunk * head_num; i += blockDim.x) {
      const long p = (i / chunk) * head_stride + (i % chunk);
      to[p] = from[p];
    }
  }
}

static int refresh_cache_check(const void* a, const void* b, const void* c, const void* d2,
                               int n_layer, int rows, int beam_size, int d, int head_num,
                               int cur_step, int max_step) {
  if (!a || !b || !c || !d2 || n_layer <= 0 || rows <= 0 || beam_size <= 0 ||
      rows % beam_size != 0 || d <= 0 || head_num <= 0 || cur_step < 0 || cur_step >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "ker_refresh_cache: bad arguments");
  if (a == c || b == d2)
    return lsh_fail(LSH_ERR_INVALID, "ker_refresh_cache: old and new cache must differ");
  if (rows * 2 > 65535) return lsh_fail(LSH_ERR_UNSUPPORTED, "ker_refresh_cache: too many rows");
  return LSH_OK;
}

int refresh_cache_i8(int n_layer, int rows_x2, hipStream_t s, const int* num_can_per_beam,
                     const int* can_idx, const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                     int8_t* v_new, long layer_offset, int beam_size, int dim_per_head,
                     int head_num, int vocab_size, int cur_step, int max_step, bool diverse,
                     int end_id) {
  if (diverse) return lsh_fail(LSH_ERR_UNSUPPORTED, "ker_refresh_cache: diverse beam search");
  if (!num_can_per_beam || !can_idx || vocab_size <= 0 || (rows_x2 & 1))
    return lsh_fail(LSH_ERR_INVALID, "ker_refresh_cache: bad arguments");
  if (int rc = refresh_cache_check(k_old, v_old, k_new, v_new, n_layer, rows_x2 / 2, beam_size,
                                   dim_per_head, head_num, cur_step, max_step))
    return rc;
  refresh_cache_kernel<false><<<dim3(n_layer, rows_x2), 256, 0, s>>>(
      num_can_per_beam, can_idx, nullptr, k_old, v_old, k_new, v_new, layer_offset, beam_size,
      dim_per_head, head_num, vocab_size, cur_step, max_step, end_id);
  return lsh_check_launch("refresh_cache_kernel<false>");
}

int refresh_cache_by_parent_i8(int n_layer, int rows, hipStream_t s, const int* parent,
                               const int8_t* k_old, const int8_t* v_old, int8_t* k_new,
                               int8_t* v_new, long layer_offset, int beam_size, int dim_per_head,
                               int head_num, int cur_step, int max_step) {
  if (!parent) return lsh_fail(LSH_ERR_INVALID, "refresh_cache_by_parent: null parent table");
  if (int rc = refresh_cache_check(k_old, v_old, k_new, v_new, n_layer, rows, beam_size,
                                   dim_per_head, head_num, cur_step, max_step))
    return rc;
  refresh_cache_kernel<true><<<dim3(n_layer, rows * 2), 256, 0, s>>>(
      nullptr, nullptr, parent, k_old, v_old, k_new, v_new, layer_offset, beam_size,
      dim_per_head, head_num, 1, cur_step, max_step, 0);
  return lsh_check_launch("refresh_cache_kernel<true>");
}

// ---------------------------------------------------------------------------------
// output writers (inference/kernels/transformerKernels.cc.cu:1707-1815)
// ---------------------------------------------------------------------------------
__global__ void write_trg_tokenid_pos_penalty_kernel(const int* __restrict__ alive_seq,
                                                     float* seq_score, int* __restrict__ output,
                                                     int max_step, int beam_size, int batch,
                                                     int out_len) {
  const int b = blockIdx.x;
  for (int t = threadIdx.x; t < out_len; t += blockDim.x)
    output[(long)b * out_len + t] = alive_seq[(long)b * beam_size * max_step + t + 1];
  if (b == 0) {
    // slot b <- score of sentence b's first beam, every read taken before the slot it
    // targets can be overwritten (chunks in ascending order, reads before writes)
    for (int c0 = 0; c0 < batch; c0 += blockDim.x) {
      const int i = c0 + threadIdx.x;
      float v = 0.f;
      if (i < batch) v = seq_score[(long)i * beam_size] - (float)i * kMinLogProb;
      __syncthreads();
      if (i < batch) seq_score[i] = v;
      __syncthreads();
    }
  }
}

__global__ void write_trg_tokenid_neg_penalty_kernel(const int* __restrict__ alive_seq,
                                                     const float* __restrict__ seq_score,
                                                     int* __restrict__ output, int max_step,
                                                     int beam_size, int end_id, int out_len) {
#pragma clang fp contract(off)
  __shared__ float red[16];
  const int b = blockIdx.x;
  float best = kFloatInfNeg;
  int res = 0;
  for (int j = 0; j < beam_size; ++j) {
    float n = 0.f;
    for (int t = threadIdx.x; t < out_len; t += blockDim.x)
      n += alive_seq[((long)b * beam_size + j) * max_step + t + 1] != end_id ? 1.f : 0.f;
    n = block_sum(n, red);
    float sc = seq_score[b * beam_size + j] - (float)b * kMinLogProb;
    sc /= (n + kSeqLenEpsilon);
    if (sc > best) {
      best = sc;
      res = j;
    }
  }
  for (int t = threadIdx.x; t < out_len; t += blockDim.x)
    output[(long)b * out_len + t] = alive_seq[((long)b * beam_size + res) * max_step + t + 1];
}

__global__ void write_topk_result_kernel(const int* __restrict__ alive_seq, float* seq_score,
                                         int* __restrict__ res_seq, int max_step, int beam_size,
                                         int end_id, int out_len) {
#pragma clang fp contract(off)
  const int r = blockIdx.x;
  for (int t = threadIdx.x; t < out_len; t += blockDim.x)
    res_seq[(long)r * out_len + t] =
        t == out_len - 1 ? end_id : alive_seq[(long)r * max_step + t + 1];
  if (threadIdx.x == 0) seq_score[r] -= (float)(r / beam_size) * kMinLogProb;
}

static int write_check(const void* a, const void* b, const void* c, int rows, int max_step,
                       int beam_size, int out_len, const char* who) {
  if (!a || !b || !c || rows <= 0 || beam_size <= 0 || out_len <= 0 || out_len + 1 > max_step) {
    lsh_fail(LSH_ERR_INVALID, who);
    return LSH_ERR_INVALID;
  }
  return LSH_OK;
}

int write_trg_tokenid_pos_penalty(const int* alive_seq, float* seq_score, int* output,
                                  int max_step, int beam_size, int batch_size, int out_len,
                                  hipStream_t s) {
  if (int rc = write_check(alive_seq, seq_score, output, batch_size, max_step, beam_size, out_len,
                           "ker_write_trg_tokenid_pos_penalty: bad arguments"))
    return rc;
  write_trg_tokenid_pos_penalty_kernel<<<batch_size, 256, 0, s>>>(
      alive_seq, seq_score, output, max_step, beam_size, batch_size, out_len);
  return lsh_check_launch("write_trg_tokenid_pos_penalty_kernel");
}

int write_trg_tokenid_neg_penalty(const int* alive_seq, const float* seq_score, int* output,
                                  int max_step, int beam_size, int vocab_size, int end_id,
                                  int batch_size, int out_len, hipStream_t s) {
  (void)vocab_size;
  if (int rc = write_check(alive_seq, seq_score, output, batch_size, max_step, beam_size, out_len,
                           "ker_write_trg_tokenid_neg_penalty: bad arguments"))
    return rc;
  write_trg_tokenid_neg_penalty_kernel<<<batch_size, 256, 0, s>>>(
      alive_seq, seq_score, output, max_step, beam_size, end_id, out_len);
  return lsh_check_launch("write_trg_tokenid_neg_penalty_kernel");
}

int write_topk_result(const int* alive_seq, float* seq_score, int* res_seq, int vocab_size,
                      int max_step, int beam_size, int end_id, int rows, int out_len,
                      hipStream_t s) {
  (void)vocab_size;
  // the last output column is the end token whatever the sequence holds, so a sampling run that
  // used every step (out_len == max_step; the reference reads one element past the row there)
  // stays inside the row
  if (int rc = write_check(alive_seq, seq_score, res_seq, rows, max_step, beam_size,
                           out_len == max_step ? out_len - 1 : out_len,
                           "ker_write_topk_result: bad arguments"))
    return rc;
  write_topk_result_kernel<<<rows, 256, 0, s>>>(alive_seq, seq_score, res_seq, max_step,
                                                beam_size, end_id, out_len);
  return lsh_check_launch("write_topk_result_kernel");
}

// ---------------------------------------------------------------------------------
// The decoder's own search step.
//
// beam_topk_kernel: one 1024-thread block per row; `beam_size` rounds of a block-wide
// arg-max over (score descending, vocabulary id ascending), each round restricted to
// the keys after the previous pick.  Output [rows, beam_size] (score, candidate id);
// a finished row proposes <eos> with its own score in slot 0 and nothing else.
// ---------------------------------------------------------------------------------
struct ScoreIdx {
  float s;
  int i;
};
// true when a comes before b: higher score, then lower id
__device__ __forceinline__ bool before(const ScoreIdx& a, const ScoreIdx& b) {
  return a.s > b.s || (a.s == b.s && a.i < b.i);
}
__device__ __forceinline__ ScoreIdx wave_first(ScoreIdx v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) {
    ScoreIdx o;
    o.s = __shfl_xor(v.s, m, 64);
    o.i = __shfl_xor(v.i, m, 64);
    if (before(o, v)) v = o;
  }
  return v;
}

constexpr int kNoCand = 0x7fffffff;

template <typename T>
__global__ void __launch_bounds__(1024)
beam_topk_kernel(const int8_t* __restrict__ logits, const T* __restrict__ logit_bias,
                 const float* __restrict__ seq_probs, const float* __restrict__ seq_score,
                 const int* __restrict__ alive_seq, float dq, float* __restrict__ top_score,
                 int* __restrict__ top_idx, int vocab, int max_step, float length_norm,
                 int cur_step, int beam_size, int end_id, int* __restrict__ num_finished) {
#pragma clang fp contract(off)
  // the merge that follows adds its finished beams to the count: it starts at zero
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *num_finished = 0;
  __shared__ float red[1024 + 32];
  __shared__ ScoreIdx wbest[16];
  const int row = blockIdx.x, t = threadIdx.x;
  const int lane = t & 63, wid = t >> 6;
  const int batch_id = row / beam_size, beam_id = row % beam_size;
  float* os = top_score + (long)row * beam_size;
  int* oi = top_idx + (long)row * beam_size;
  if (cur_step != 0 && alive_seq[(long)row * max_step + cur_step] == end_id) {
    if (t < beam_size) {
      os[t] = t == 0 ? seq_score[row] : -INFINITY;
      oi[t] = t == 0 ? end_id + beam_id * vocab : kNoCand;
    }
    return;
  }
  const int8_t* lr = logits + (long)row * vocab;
  const RowStats st = row_stats(lr, logit_bias, vocab, dq, 0, 0, red);
  const float base = seq_probs[row] - logf(st.sum_exp) - st.max_logit;
  ScoreIdx prev;
  prev.s = INFINITY;
  prev.i = -1;
  for (int k = 0; k < beam_size; ++k) {
    ScoreIdx best;
    best.s = -INFINITY;
    best.i = kNoCand;
    for (int v = t; v < vocab; v += 1024) {
      ScoreIdx c;
      c.s = cand_score(logit_of(lr, logit_bias, v, dq), base, length_norm, batch_id);
      c.i = v;
      if (before(prev, c) && before(c, best)) best = c;
    }
    best = wave_first(best);
    __syncthreads();
    if (lane == 0) wbest[wid] = best;
    __syncthreads();
    best = wbest[0];
    for (int w2 = 1; w2 < 16; ++w2)
      if (before(wbest[w2], best)) best = wbest[w2];
    if (t == 0) {
      os[k] = best.i == kNoCand ? -INFINITY : best.s;
      oi[k] = best.i == kNoCand ? kNoCand : beam_id * vocab + best.i;
    }
    prev = best;
  }
}

// The same selection for vocabularies of up to 32 * 1024 entries with the row's logits kept
// in registers: thread t loads its ids t, t + 1024, ... once (all loads in flight together)
// and every later pass -- maximum, sum of exponentials in the same ascending order, the
// `beam_size` arg-max rounds -- works on registers.  Same arithmetic and the same order as
// beam_topk_kernel, hence the same bits.  VEC (vocab % 16 == 0, 16-byte aligned rows):
// thread t owns ids 16 t .. 16 t + 15 of each 16384-id half instead and reads them with
// 16-byte loads; the sum of exponentials then runs in another order (a last-place
// difference of the log-sum-exp, shared by all candidates of the row).
template <typename T, bool VEC>
__global__ void __launch_bounds__(1024)
beam_topk_reg_kernel(const int8_t* __restrict__ logits, const T* __restrict__ logit_bias,
                     const float* __restrict__ seq_probs, const float* __restrict__ seq_score,
                     const int* __restrict__ alive_seq, float dq, float* __restrict__ top_score,
                     int* __restrict__ top_idx, int vocab, int max_step, float length_norm,
                     int cur_step, int beam_size, int end_id, int* __restrict__ num_finished) {
#pragma clang fp contract(off)
  // the merge that follows adds its finished beams to the count: it starts at zero
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *num_finished = 0;
  constexpr int NI = 32;
  __shared__ float red_max[16], red_sum[16];
  __shared__ unsigned long long wbest[2][16];  // per-wavefront best key, double-buffered by round
  const int row = blockIdx.x, t = threadIdx.x;
  const int lane = t & 63, wid = t >> 6;
  const int batch_id = row / beam_size, beam_id = row % beam_size;
  float* os = top_score + (long)row * beam_size;
  int* oi = top_idx + (long)row * beam_size;
  if (cur_step != 0 && alive_seq[(long)row * max_step + cur_step] == end_id) {
    if (t < beam_size) {
      os[t] = t == 0 ? seq_score[row] : -INFINITY;
      oi[t] = t == 0 ? end_id + beam_id * vocab : kNoCand;
    }
    return;
  }
  const int8_t* lr = logits + (long)row * vocab;
  float lg[NI];
  auto id_of = [&](int i) { return VEC ? (i >> 4) * 16384 + 16 * t + (i & 15) : t + 1024 * i; };
  if (VEC) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int v0 = h * 16384 + 16 * t;
      if (v0 < vocab) {
        const uint4 w = *reinterpret_cast<const uint4*>(lr + v0);
        float b[16];
        ld4(logit_bias, v0, *reinterpret_cast<float(*)[4]>(b));
        ld4(logit_bias, v0 + 4, *reinterpret_cast<float(*)[4]>(b + 4));
        ld4(logit_bias, v0 + 8, *reinterpret_cast<float(*)[4]>(b + 8));
        ld4(logit_bias, v0 + 12, *reinterpret_cast<float(*)[4]>(b + 12));
        const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 0; e < 16; ++e)
          lg[h * 16 + e] = (float)unpack_i8(ws[e >> 2], e & 3) * dq + b[e];
      } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) lg[h * 16 + e] = 0.f;
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int v = t + 1024 * i;
      lg[i] = v < vocab ? logit_of(lr, logit_bias, v, dq) : 0.f;
    }
  }
  float tmax = kFloatInfNeg;
#pragma unroll
  for (int i = 0; i < NI; ++i)
    if (id_of(i) < vocab) tmax = fmaxf(tmax, lg[i]);
  const float max_logit = block_max_dpp(tmax, red_max);
  float se = 0.f;
#pragma unroll
  for (int i = 0; i < NI; ++i)
    if (id_of(i) < vocab) se += __expf(fmaxf(lg[i] - max_logit, kLogitThreshMin));
  const float sum_exp = block_sum_dpp(se, red_sum);
  const float base = seq_probs[row] - logf(sum_exp) - max_logit;
#pragma unroll
  for (int i = 0; i < NI; ++i) lg[i] = cand_score(lg[i], base, length_norm, batch_id);
  // A candidate is one 64-bit key: the score as an order-preserving integer above
  // 2^31 - 1 - id, so "higher score first, lower id on ties" is an integer maximum.  A thread
  // keeps the largest of its own keys that is below the last pick; a round is a block-wide
  // maximum over these -- DPP permutations and lane reads inside a wavefront, one barrier
  // and 16 LDS reads across the workgroup -- and only the thread that owned the pick looks
  // through its registers again (every other thread's key is still below it).
  auto key_of = [&](int i) -> unsigned long long {
    const int id = id_of(i);
    if (id >= vocab) return 0ull;
    unsigned u = __builtin_bit_cast(unsigned, lg[i] + 0.f);  // -0 -> +0
    u ^= (u >> 31) ? 0xffffffffu : 0x80000000u;
    return ((unsigned long long)u << 32) | (unsigned)(0x7fffffff - id);
  };
  auto my_best_below = [&](unsigned long long bound) {
    unsigned long long best = 0ull;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const unsigned long long c = key_of(i);
      if (c < bound && c > best) best = c;
    }
    return best;
  };
  auto umax64 = [](unsigned long long a, unsigned long long b) { return a > b ? a : b; };
  auto dpp64 = [](unsigned long long x, auto ctrl) {
    const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)x, decltype(ctrl)::value, 0xf, 0xf, false);
    const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)(x >> 32), decltype(ctrl)::value, 0xf, 0xf, false);
    return ((unsigned long long)hi << 32) | lo;
  };
  auto lane64 = [](unsigned long long x, int l) {
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)x, l);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(x >> 32), l);
    return ((unsigned long long)hi << 32) | lo;
  };
  unsigned long long mine = my_best_below(~0ull);
  for (int k = 0; k < beam_size; ++k) {
    unsigned long long best = mine;
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppXor1>()));
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppXor2>()));
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppHalfMirror>()));
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppMirror>()));
    best = umax64(umax64(lane64(best, 0), lane64(best, 16)), umax64(lane64(best, 32), lane64(best, 48)));
    unsigned long long* wb = wbest[k & 1];
    if (lane == 0) wb[wid] = best;
    __syncthreads();
    best = wb[0];
#pragma unroll
    for (int w2 = 1; w2 < 16; ++w2) best = umax64(best, wb[w2]);
    if (t == 0) {
      // key 0: no candidate left
      unsigned u = (unsigned)(best >> 32);
      u ^= (u >> 31) ? 0x80000000u : 0xffffffffu;
      os[k] = best == 0ull ? -INFINITY : __builtin_bit_cast(float, u);
      oi[k] = best == 0ull ? kNoCand : beam_id * vocab + (0x7fffffff - (int)(unsigned)best);
    }
    if (best == mine && best != 0ull) mine = my_best_below(best);
  }
}

// The per-row top-k dealt to P workgroups per row (vocabularies of up to 32 * 1024 ids, VEC
// layout): beam_topk_reg_kernel is bound by vector instructions -- a row's 32 K logits cost
// about 45 instructions each and one workgroup keeps them all on one compute unit, 64 rows on
// 64 of the 256 -- so a row's ids are cut into P <= 4 parts of at most 8192 and the top-k runs
// as rows x P workgroups of 512 threads (16 ids per thread and part).  Every workgroup of a row
// computes the row's maximum and sum of exponentials itself, from all of the row (the one-pass
// sums of beam_topk_reg_kernel in another order; a separate statistics launch ahead of it cost
// more than the repeated arithmetic), then the scores of its own part's ids and the part's
// best beam_size by the same 64-bit keys.
// The merge then reads P * beam_size proposals per row instead of beam_size: a row's best
// beam_size by (score, id) are among the union of its parts' best beam_size by (score, id), so
// the beams chosen are the same.
template <typename T>
__device__ __forceinline__ void beam_part_load(const int8_t* __restrict__ lr,
                                               const T* __restrict__ logit_bias, int lo, int hi,
                                               float dq, float (&lg)[16]) {
#pragma clang fp contract(off)
  // thread t owns ids lo + 16 t .. + 15: 512 threads, one 16-byte piece each (two wavefronts
  // per SIMD take turns; with 32 ids per thread and one wavefront per SIMD every dependent
  // instruction waits out its latency and the kernel takes twice as long)
  const int v0 = lo + 16 * (int)threadIdx.x;
  if (v0 < hi) {
    const uint4 w = *reinterpret_cast<const uint4*>(lr + v0);
    float b[16];
    ld4(logit_bias, v0, *reinterpret_cast<float(*)[4]>(b));
    ld4(logit_bias, v0 + 4, *reinterpret_cast<float(*)[4]>(b + 4));
    ld4(logit_bias, v0 + 8, *reinterpret_cast<float(*)[4]>(b + 8));
    ld4(logit_bias, v0 + 12, *reinterpret_cast<float(*)[4]>(b + 12));
    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int e = 0; e < 16; ++e) lg[e] = (float)unpack_i8(ws[e >> 2], e & 3) * dq + b[e];
  } else {
#pragma unroll
    for (int e = 0; e < 16; ++e) lg[e] = 0.f;
  }
}

constexpr int kBeamPartIds = 8192;  // ids of a part, at most (a multiple of 16: parts stay aligned)

template <typename T>
__global__ void __launch_bounds__(512)
beam_topk_part_kernel(const int8_t* __restrict__ logits, const T* __restrict__ logit_bias,
                      const float* __restrict__ seq_probs, const float* __restrict__ seq_score,
                      const int* __restrict__ alive_seq, float dq, float* __restrict__ top_score,
                      int* __restrict__ top_idx, int vocab, int max_step, float length_norm,
                      int cur_step, int beam_size, int end_id, int* __restrict__ num_finished) {
#pragma clang fp contract(off)
  // the merge that follows adds its finished beams to the count: it starts at zero
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *num_finished = 0;
  __shared__ unsigned long long wbest[2][8];
  __shared__ float red_max[16], red_sum[16];
  const int part = blockIdx.x, row = blockIdx.y, P = gridDim.x, t = threadIdx.x;
  const int lane = t & 63, wid = t >> 6;
  const int batch_id = row / beam_size, beam_id = row % beam_size;
  float* os = top_score + ((long)row * P + part) * beam_size;
  int* oi = top_idx + ((long)row * P + part) * beam_size;
  if (cur_step != 0 && alive_seq[(long)row * max_step + cur_step] == end_id) {
    // a finished beam proposes itself once (part 0, slot 0)
    if (t < beam_size) {
      const bool self = part == 0 && t == 0;
      os[t] = self ? seq_score[row] : -INFINITY;
      oi[t] = self ? end_id + beam_id * vocab : kNoCand;
    }
    return;
  }
  const int lo = part * kBeamPartIds, hi = min(lo + kBeamPartIds, vocab);
  // the row's maximum and sum of exponentials: every workgroup of the row reads all of it (the
  // other parts' logits come from L2), so no workgroup waits for another
  float all[4][16];
#pragma unroll
  for (int p = 0; p < 4; ++p)
    beam_part_load(logits + (long)row * vocab, logit_bias, p * kBeamPartIds,
                   min((p + 1) * kBeamPartIds, vocab), dq, all[p]);
  float tmax = kFloatInfNeg;
#pragma unroll
  for (int p = 0; p < 4; ++p)
    if (p * kBeamPartIds + 16 * t < vocab) {
#pragma unroll
      for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, all[p][i]);
    }
  const float max_logit = block_max_dpp(tmax, red_max);
  float se = 0.f;
#pragma unroll
  for (int p = 0; p < 4; ++p)
    if (p * kBeamPartIds + 16 * t < vocab) {
#pragma unroll
      for (int i = 0; i < 16; ++i) se += __expf(fmaxf(all[p][i] - max_logit, kLogitThreshMin));
    }
  const float sum_exp = block_sum_dpp(se, red_sum);
  float lg[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
    lg[i] = part == 0 ? all[0][i] : part == 1 ? all[1][i] : part == 2 ? all[2][i] : all[3][i];
  const float base = seq_probs[row] - logf(sum_exp) - max_logit;
#pragma unroll
  for (int i = 0; i < 16; ++i) lg[i] = cand_score(lg[i], base, length_norm, batch_id);
  auto id_of = [&](int i) { return lo + 16 * t + i; };
  auto key_of = [&](int i) -> unsigned long long {
    const int id = id_of(i);
    if (id >= hi) return 0ull;
    unsigned u = __builtin_bit_cast(unsigned, lg[i] + 0.f);  // -0 -> +0
    u ^= (u >> 31) ? 0xffffffffu : 0x80000000u;
    return ((unsigned long long)u << 32) | (unsigned)(0x7fffffff - id);
  };
  auto my_best_below = [&](unsigned long long bound) {
    unsigned long long best = 0ull;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const unsigned long long c = key_of(i);
      if (c < bound && c > best) best = c;
    }
    return best;
  };
  auto umax64 = [](unsigned long long a, unsigned long long b) { return a > b ? a : b; };
  auto dpp64 = [](unsigned long long x, auto ctrl) {
    const unsigned l = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)x, decltype(ctrl)::value, 0xf, 0xf, false);
    const unsigned h = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)(x >> 32), decltype(ctrl)::value, 0xf, 0xf, false);
    return ((unsigned long long)h << 32) | l;
  };
  auto lane64 = [](unsigned long long x, int l) {
    const unsigned lo32 = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)x, l);
    const unsigned hi32 = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(x >> 32), l);
    return ((unsigned long long)hi32 << 32) | lo32;
  };
  unsigned long long mine = my_best_below(~0ull);
  for (int k = 0; k < beam_size; ++k) {
    unsigned long long best = mine;
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppXor1>()));
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppXor2>()));
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppHalfMirror>()));
    best = umax64(best, dpp64(best, std::integral_constant<int, kDppMirror>()));
    best = umax64(umax64(lane64(best, 0), lane64(best, 16)), umax64(lane64(best, 32), lane64(best, 48)));
    unsigned long long* wb = wbest[k & 1];
    if (lane == 0) wb[wid] = best;
    __syncthreads();
    best = umax64(umax64(umax64(wb[0], wb[1]), umax64(wb[2], wb[3])),
                  umax64(umax64(wb[4], wb[5]), umax64(wb[6], wb[7])));
    if (t == 0) {
      unsigned u = (unsigned)(best >> 32);
      u ^= (u >> 31) ? 0x80000000u : 0xffffffffu;
      os[k] = best == 0ull ? -INFINITY : __builtin_bit_cast(float, u);
      oi[k] = best == 0ull ? kNoCand : beam_id * vocab + (0x7fffffff - (int)(unsigned)best);
    }
    if (best == mine && best != 0ull) mine = my_best_below(best);
  }
}

// beam_merge_kernel: one workgroup of one wavefront per sentence (more than 1024 sentences are
// dealt round-robin).  Picks the sentence's best `beam_size` of its
// beam_size * beam_size * parts proposals in (score descending, candidate id ascending) order
// and applies ker_refresh_result to them (inference/kernels/transformerKernels.cc.cu:
// 1398-1463): new sequences, summed log-probabilities of live beams, scores of
// finished ones, the finished count (added to *num_finished, which the top-k kernel ahead of
// it cleared), plus the parent table for the cache reorder.
__global__ void __launch_bounds__(64)
beam_merge_kernel(const float* __restrict__ top_score, const int* __restrict__ top_idx,
                  const int* __restrict__ old_alive_seq, int* __restrict__ new_alive_seq,
                  float* __restrict__ seq_probs, float* __restrict__ seq_score,
                  int* __restrict__ parent, int* __restrict__ num_finished, int batch,
                  int beam_size, int vocab, int max_step, int cur_step, float length_norm,
                  int end_id, int parts) {
#pragma clang fp contract(off)
  // grid: a workgroup of one wavefront per sentence (16 sentences as the 16 wavefronts of one
  // workgroup took turns on one compute unit's SIMDs: four times the time per instruction)
  __shared__ int seq_lds[1][512];  // the sentence's old sequences (beam_size * max_step <= 512)
  const int lane = threadIdx.x & 63, wid = 0;
  const int nw = gridDim.x;
  const int ncand = beam_size * beam_size * parts;  // proposals of a sentence
  int finished = 0;
  // applies one pick (ker_refresh_result): the new sequence, then probability or score
  auto apply = [&](int b, int j, float score, int idx) {
    // a sentence always has at least beam_size proposals; guard the indices anyway
    const int ori = idx == kNoCand ? end_id : idx;
    int can_beam = ori / vocab;
    const int can_vocab = ori % vocab;
    if (can_beam >= beam_size) can_beam = 0;
    const int* from = old_alive_seq + ((long)b * beam_size + can_beam) * max_step;
    int* to = new_alive_seq + ((long)b * beam_size + j) * max_step;
    for (int t = lane; t < max_step; t += 64)
      to[t] = t > cur_step + 1 ? end_id : (t == cur_step + 1 ? can_vocab : from[t]);
    if (lane == 0) {
      if (can_vocab != end_id) {
        seq_probs[b * beam_size + j] = (score - (float)b * kMinLogProb) / length_norm;
        parent[b * beam_size + j] = can_beam;
      } else {
        seq_score[b * beam_size + j] = score;
        parent[b * beam_size + j] = -1;
        ++finished;
      }
    }
  };
  if (ncand <= 256) {
    // up to four proposals per lane, held in registers as 64-bit keys (score as an
    // order-preserving integer above 2^31 - 1 - id: "higher score first, lower id on ties" is
    // an integer maximum); the picks are made first, without touching memory, then applied
    auto dpp64 = [](unsigned long long x, auto ctrl) {
      const unsigned l = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)x, decltype(ctrl)::value, 0xf, 0xf, false);
      const unsigned h = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)(x >> 32), decltype(ctrl)::value, 0xf, 0xf, false);
      return ((unsigned long long)h << 32) | l;
    };
    auto lane64 = [](unsigned long long x, int l) {
      const unsigned lo32 = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)x, l);
      const unsigned hi32 = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(x >> 32), l);
      return ((unsigned long long)hi32 << 32) | lo32;
    };
    auto umax64 = [](unsigned long long a, unsigned long long b) { return a > b ? a : b; };
    const int total = beam_size * max_step;
    const bool staged = total <= 512;
    for (int b = blockIdx.x; b < batch; b += nw) {
      const float* cs = top_score + (long)b * ncand;
      const int* ci = top_idx + (long)b * ncand;
      // the sentence's old sequences are requested together with the proposals and parked in
      // LDS: the new sequences then cost no second trip to memory after the picks are known
      int olds[8];
      if (staged) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
          olds[u] = old_alive_seq[(long)b * total + min(lane + 64 * u, total - 1)];
      }
      unsigned long long key[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int c = min(lane + 64 * q, ncand - 1);
        const float sc = cs[c];
        const int id = ci[c];
        unsigned u = __builtin_bit_cast(unsigned, sc + 0.f);
        u ^= (u >> 31) ? 0xffffffffu : 0x80000000u;
        key[q] = (lane + 64 * q < ncand && id != kNoCand)
                     ? (((unsigned long long)u << 32) | (unsigned)(0x7fffffff - id)) : 0ull;
      }
      unsigned long long bound = ~0ull, won = 0ull;  // lane j keeps pick j
      for (int j = 0; j < beam_size; ++j) {
        unsigned long long best = 0ull;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (key[q] < bound && key[q] > best) best = key[q];
        best = umax64(best, dpp64(best, std::integral_constant<int, kDppXor1>()));
        best = umax64(best, dpp64(best, std::integral_constant<int, kDppXor2>()));
        best = umax64(best, dpp64(best, std::integral_constant<int, kDppHalfMirror>()));
        best = umax64(best, dpp64(best, std::integral_constant<int, kDppMirror>()));
        best = umax64(umax64(lane64(best, 0), lane64(best, 16)), umax64(lane64(best, 32), lane64(best, 48)));
        if (lane == j) won = best;
        bound = best;  // 0 once nothing is left: no key lies below it
      }
      if (staged) {
#pragma unroll
        for (int u = 0; u < 8; ++u) seq_lds[wid][lane + 64 * u] = olds[u];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      // the picks applied (ker_refresh_result): beam by beam, with the pick, its source beam and
      // its token in scalar registers (one division per beam, none per element), the old
      // sequence read from LDS; then probabilities and scores, a lane per beam
      for (int j = 0; j < beam_size; ++j) {
        const unsigned long long k = lane64(won, j);
        const int ori = k == 0ull ? end_id : 0x7fffffff - (int)(unsigned)k;
        int can_beam = ori / vocab;
        const int can_vocab = ori - can_beam * vocab;
        if (can_beam >= beam_size) can_beam = 0;
        const int* from = old_alive_seq + ((long)b * beam_size + can_beam) * max_step;
        int* to = new_alive_seq + ((long)b * beam_size + j) * max_step;
        for (int t = lane; t < max_step; t += 64) {
          const int old = staged ? seq_lds[wid][can_beam * max_step + t] : from[t];
          to[t] = t > cur_step + 1 ? end_id : (t == cur_step + 1 ? can_vocab : old);
        }
      }
      if (lane < beam_size) {
        const int j = lane;
        const unsigned long long k = won;
        unsigned u = (unsigned)(k >> 32);
        u ^= (u >> 31) ? 0x80000000u : 0xffffffffu;
        const float score = k == 0ull ? -INFINITY : __builtin_bit_cast(float, u);
        const int ori = k == 0ull ? end_id : 0x7fffffff - (int)(unsigned)k;
        if (ori % vocab != end_id) {
          int can_beam = ori / vocab;
          if (can_beam >= beam_size) can_beam = 0;
          seq_probs[b * beam_size + j] = (score - (float)b * kMinLogProb) / length_norm;
          parent[b * beam_size + j] = can_beam;
        } else {
          seq_score[b * beam_size + j] = score;
          parent[b * beam_size + j] = -1;
          ++finished;
        }
      }
    }
  } else {
    for (int b = blockIdx.x; b < batch; b += nw) {
      const float* cs = top_score + (long)b * ncand;
      const int* ci = top_idx + (long)b * ncand;
      ScoreIdx prev;
      prev.s = INFINITY;
      prev.i = -1;
      for (int j = 0; j < beam_size; ++j) {
        ScoreIdx best;
        best.s = -INFINITY;
        best.i = kNoCand;
        for (int c = lane; c < ncand; c += 64) {
          ScoreIdx x;
          x.s = cs[c];
          x.i = ci[c];
          if (x.i != kNoCand && before(prev, x) && before(x, best)) best = x;
        }
        best = wave_first(best);
        prev = best;
        apply(b, j, best.s, best.i);
      }
    }
  }
  for (int d = 32; d > 0; d >>= 1) finished += __shfl_xor(finished, d);  // lanes count their own picks
  if (lane == 0 && finished != 0) atomicAdd(num_finished, finished);  // cleared by the top-k kernel
}

// 4-byte words of the optional second workspace with which the per-row top-k is dealt to
// several workgroups per row (0: the shape does not use one): per (row, part) beam_size
// proposals (score, id).
size_t beam_search_step_workspace_words(int batch_size, int beam_size, int vocab_size) {
  if (batch_size <= 0 || beam_size <= 0 || vocab_size <= kBeamPartIds || vocab_size > 32 * 1024 ||
      vocab_size % 16 != 0)
    return 0;
  const size_t parts = (size_t)(vocab_size + kBeamPartIds - 1) / kBeamPartIds;
  return (size_t)batch_size * beam_size * parts * 2 * (size_t)beam_size;
}

template <typename T>
int beam_search_step_i8I(const int8_t* logits, const T* logit_bias, float* seq_probs,
                         float* seq_score, const int* old_alive_seq, int* new_alive_seq,
                         float* top_score, int* top_idx, int* parent, int* num_finished,
                         float dequant_scale, int vocab_size, int max_step, float length_norm,
                         int cur_step, int batch_size, int beam_size, int end_id, hipStream_t s,
                         float* part_ws, size_t part_ws_words) {
  if (!logits || !logit_bias || !seq_probs || !seq_score || !old_alive_seq || !new_alive_seq ||
      !top_score || !top_idx || !parent || !num_finished || vocab_size <= 0 || batch_size <= 0 ||
      max_step <= 0 || cur_step < 0 || cur_step + 1 >= max_step)
    return lsh_fail(LSH_ERR_INVALID, "beam_search_step: bad arguments");
  if (beam_size < 1 || beam_size > 32 || (beam_size & (beam_size - 1)))
    return lsh_fail(LSH_ERR_INVALID, "wrong beam_size, should be 1, 2, 4, 8, 16 or 32");
  if (old_alive_seq == new_alive_seq)
    return lsh_fail(LSH_ERR_INVALID, "beam_search_step: the sequence buffers must differ");
  if ((long)beam_size * vocab_size > 0x7ffffffe)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "beam_search_step: beam_size * vocab_size overflows");
  const bool vec = vocab_size % 16 == 0 &&
                   ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(logit_bias)) &
                    15u) == 0;
  const int rows = batch_size * beam_size;
  const size_t need = beam_search_step_workspace_words(batch_size, beam_size, vocab_size);
  int parts = 1;
  if (vec && part_ws != nullptr && need != 0 && part_ws_words >= need && rows <= 65535 &&
      (reinterpret_cast<uintptr_t>(part_ws) & 7u) == 0) {
    // the row's ids dealt to several workgroups
    parts = (vocab_size + kBeamPartIds - 1) / kBeamPartIds;
    float* p_score = part_ws;
    int* p_idx = reinterpret_cast<int*>(p_score + (size_t)rows * parts * beam_size);
    beam_topk_part_kernel<T><<<dim3(parts, rows), 512, 0, s>>>(
        logits, logit_bias, seq_probs, seq_score, old_alive_seq, dequant_scale, p_score, p_idx,
        vocab_size, max_step, length_norm, cur_step, beam_size, end_id, num_finished);
    if (int rc = lsh_check_launch("beam_topk_part_kernel")) return rc;
    top_score = p_score;
    top_idx = p_idx;
  } else if (vocab_size <= 32 * 1024 && vec)
    beam_topk_reg_kernel<T, true><<<batch_size * beam_size, 1024, 0, s>>>(
        logits, logit_bias, seq_probs, seq_score, old_alive_seq, dequant_scale, top_score,
        top_idx, vocab_size, max_step, length_norm, cur_step, beam_size, end_id, num_finished);
  else if (vocab_size <= 32 * 1024)
    beam_topk_reg_kernel<T, false><<<batch_size * beam_size, 1024, 0, s>>>(
        logits, logit_bias, seq_probs, seq_score, old_alive_seq, dequant_scale, top_score,
        top_idx, vocab_size, max_step, length_norm, cur_step, beam_size, end_id, num_finished);
  else
    beam_topk_kernel<T><<<batch_size * beam_size, 1024, 0, s>>>(
        logits, logit_bias, seq_probs, seq_score, old_alive_seq, dequant_scale, top_score,
        top_idx, vocab_size, max_step, length_norm, cur_step, beam_size, end_id, num_finished);
  if (int rc = lsh_check_launch("beam_topk_kernel")) return rc;
  beam_merge_kernel<<<batch_size < 1024 ? batch_size : 1024, 64, 0, s>>>(top_score, top_idx, old_alive_seq, new_alive_seq,
                                       seq_probs, seq_score, parent, num_finished, batch_size,
                                       beam_size, vocab_size, max_step, cur_step, length_norm,
                                       end_id, parts);
  return lsh_check_launch("beam_merge_kernel");
}
template int beam_search_step_i8I<float>(const int8_t*, const float*, float*, float*, const int*,
                                         int*, float*, int*, int*, int*, float, int, int, float,
                                         int, int, int, int, hipStream_t, float*, size_t);
template int beam_search_step_i8I<__half>(const int8_t*, const __half*, float*, float*, const int*,
                                          int*, float*, int*, int*, int*, float, int, int, float,
                                          int, int, int, int, hipStream_t, float*, size_t);

// ---------------------------------------------------------------------------------
// The search step for callers that cannot allocate device memory (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc).  The proposals of the per-row
// top-k -- the workspace that beam_search_step_i8I takes as top_score / top_idx -- live in
// a file-scope device array instead.  Every GPU holds its own copy of the array at its own
// address: the address is asked for once per device, with that device current, and host
// code only ever uses the pointer it got back, never the array's name.  All calls on one
// GPU share that GPU's array, so calls that overlap in time on one GPU race; nothing in
// it has to start at zero (the top-k kernels write every slot the merge reads).
// ---------------------------------------------------------------------------------
constexpr int kStaticBeamEntries = 65536;  // batch_size * beam_size * beam_size, at most
constexpr int kStaticBeamDevices = 64;
static __device__ __align__(256) unsigned char scratch[(size_t)kStaticBeamEntries * 8];
static std::mutex g_scratch_mutex;
static unsigned char* g_scratch_ptr[kStaticBeamDevices] = {};

static int scratch_of_current_device(unsigned char** out) {
  int dev = -1;
  if (int rc = lsh_check_hip(hipGetDevice(&dev), "hipGetDevice(beam_search_step_noalloc)")) return rc;
  if (dev < 0 || dev >= kStaticBeamDevices)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "beam_search_step_noalloc: device index out of range");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    if (int rc = lsh_check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)),
                               "hipGetSymbolAddress(beam_search_step_noalloc)"))
      return rc;
    if (!p) return lsh_fail(LSH_ERR_HIP, "beam_search_step_noalloc: null scratch address");
    g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
  }
  *out = g_scratch_ptr[dev];
  return LSH_OK;
}

int beam_search_step_noalloc_i8I_f16(const int8_t* logits, const __half* logit_bias,
                                     float* seq_probs, float* seq_score, const int* old_alive_seq,
                                     int* new_alive_seq, int* parent, int* num_finished,
                                     float dequant_scale, int vocab_size, int max_step,
                                     float length_norm, int cur_step, int batch_size, int beam_size,
                                     int end_id, hipStream_t s) {
  if (batch_size <= 0 || beam_size < 1 || beam_size > 32)
    return lsh_fail(LSH_ERR_INVALID, "beam_search_step_noalloc: bad batch_size or beam_size");
  if ((long)batch_size * beam_size * beam_size > kStaticBeamEntries)
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "beam_search_step_noalloc: batch_size * beam_size^2 exceeds the 65536 proposals "
                    "of the static workspace; use lsh_beam_search_step_i8I with a caller workspace");
  unsigned char* ws = nullptr;
  if (int rc = scratch_of_current_device(&ws)) return rc;
  float* top_score = reinterpret_cast<float*>(ws);
  int* top_idx = reinterpret_cast<int*>(ws + (size_t)kStaticBeamEntries * 4);
  return beam_search_step_i8I<__half>(logits, logit_bias, seq_probs, seq_score, old_alive_seq,
                                      new_alive_seq, top_score, top_idx, parent, num_finished,
                                      dequant_scale, vocab_size, max_step, length_norm, cur_step,
                                      batch_size, beam_size, end_id, s, nullptr, 0);
}

}  // namespace lsh
