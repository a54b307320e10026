// Token sampling of the int8 encoder-decoder model: ker_topk_sample_i8I<k> and
// ker_topp_sample_i8I of inference/kernels/transformerKernels_int8.cc.cu:1908-2290, as they act
// with the 1024 threads per block the decoder launches them with
// (inference/model/quant_decoder.cc.cu:952-998, 1101-1130).
//
// Against the GPT kernels of the same names (gpt_kernels.hip) a logit here is
// float(code) * dequant_scale + logit_bias[id], so nothing can run on the int8 codes alone:
// thread t walks the ids t, t + 1024, ... (its class) in float.  The ids stay in place in
// `ids` [rows, max_step]: a row whose last token is the end token gets another end token and
// leaves the unfinished flag alone; otherwise the token goes to column cur_len and the flag is
// set unless it is the end token.
//   k == 1   the first id of the largest logit (the reference lets every thread that holds the
//            maximum store its id: a race)
//   k > 1    threshold = rough k-th largest class maximum (kernels/common.h:118-137), one
//            candidate per class at or above it, soft-max over the candidates, one uniform number
//   top-p    threshold = the smallest class maximum inside the nucleus.  The reference forms
//            the class maximum as fmaxf(m, code * scale) + bias inside its loop (:2136-2137, the
//            bias of every id of the class is added up) and compares with a threshold that only
//            its last thread assigns (:2160-2166); built is what the code intends: class maxima
//            of code * scale + bias in descending order, exps, inclusive prefix, and the nucleus
//            is the longest prefix whose exp-sum stays within p of the total (at least the
//            largest).  The prefix of a class is summed over the classes before it in that order
//            (larger maximum, or equal maximum and lower thread).
// The product and the sum of a logit are rounded separately (no FMA contraction), so that a
// logit has one value wherever it is formed.
#include "ls_device.h"
#include "ls_launch.h"
#include "sample_common.h"

#include <string>

namespace lsh {

namespace {

constexpr float kLogitThreshMin = -64.f;  // inference/kernels/transformerKernels.h:11

template <typename T>
__device__ __forceinline__ float biased_logit(const int8_t* __restrict__ lr,
                                              const T* __restrict__ bias, int v, float scale) {
#pragma clang fp contract(off)
  const float prod = (float)lr[v] * scale;
  return prod + TT<T>::ld(bias, v);
}

// One row; every thread returns the chosen id.  k == 1: arg-max, k > 1: top-k, k == 0: top-p.
template <typename T>
__device__ int dec_sample_row(const int8_t* __restrict__ lr, const T* __restrict__ bias, int vocab,
                              int k, float p, float scale, SampleState* st, SampleShared& sh) {
#pragma clang fp contract(off)
  const int t = threadIdx.x;
  float* cmax = reinterpret_cast<float*>(sh.cls);  // class maxima; -inf = empty class
  float m = -INFINITY;
  for (int v = t; v < vocab; v += kSampleThreads) m = fmaxf(m, biased_logit(lr, bias, v, scale));
  if (t == 0 && k != 1) sh.x = sample_draw_uniform(st);
  const float gmax = block_max(m, sh.red);
  if (k == 1) {
    int first = vocab;
    for (int v = t; v < vocab; v += kSampleThreads)
      if (biased_logit(lr, bias, v, scale) == gmax) {
        first = v;
        break;
      }
    return vocab - (int)block_max((float)(vocab - first), sh.red);  // ids < 2^20: exact in float
  }
  cmax[t] = m;
  __syncthreads();
  float thr;
  if (k > 0) {
    float* warp_max = reinterpret_cast<float*>(sh.hist);
    if (t < 32) {
      float w = cmax[32 * t];
      for (int l = 1; l < 32; ++l) w = fmaxf(w, cmax[32 * t + l]);
      warp_max[t] = w;
    }
    __syncthreads();
    if (t == 0) {
      float best = INFINITY;
      for (int g = 0; g < k; ++g) {
        float w = warp_max[g];
        for (int j = g + k; j < 32; j += k) w = fmaxf(w, warp_max[j]);
        best = fminf(best, w);
      }
      sh.pf[0] = best;
    }
    __syncthreads();
    thr = sh.pf[0];
    __syncthreads();
  } else {
    const float e = expf(fmaxf(m - gmax, kLogitThreshMin));  // an empty class: exp(-64)
    sh.pf[t] = e;
    const float total = block_sum(e, sh.red);  // (its barriers publish pf)
    float before = 0.f;
    for (int u = 0; u < kSampleThreads; ++u) {
      const float mu = cmax[u];
      if (mu > m || (mu == m && u < t)) before += sh.pf[u];
    }
    const bool inside = m > -INFINITY && before + e <= p * total;
    // the smallest maximum inside the nucleus; none inside: the largest maximum
    thr = -block_max(inside ? -m : -gmax, sh.red);
    __syncthreads();
  }
  float ex = -INFINITY;
  int my_id = vocab;
  for (int v = t; v < vocab; v += kSampleThreads) {
    const float lg = biased_logit(lr, bias, v, scale);
    const float le = expf(fmaxf(lg - gmax, kLogitThreshMin));
    if (lg >= thr && le > ex) {
      ex = le;
      my_id = v;
    }
  }
  if (my_id == vocab) ex = 0.f;
  return sample_pick(ex, my_id, sh);
}

template <typename T>
__global__ void __launch_bounds__(kSampleThreads)
dec_sample_kernel(const int8_t* __restrict__ logits, const T* __restrict__ bias, int* ids,
                  int vocab, int max_step, int cur_len, int logits_seq_len, int* unfinished,
                  int eos_id, int k, float p, float scale, SampleState* st) {
  __shared__ SampleShared sh;
  const int b = blockIdx.x;
  const long last = (long)b * max_step + cur_len - 1;
  if (cur_len > 1 && ids[last] == eos_id) {
    if (threadIdx.x == 0) ids[last + 1] = eos_id;
    return;
  }
  const int8_t* lr = logits + ((long)b * logits_seq_len + logits_seq_len - 1) * vocab;
  const int tok = dec_sample_row<T>(lr, bias, vocab, k, p, scale, st ? st + b : nullptr, sh);
  if (threadIdx.x == 0) {
    if (tok != eos_id) unfinished[0] = 1;
    ids[last + 1] = tok;
  }
}

template <typename T>
int dec_sample(const char* who, int rows, int cur_len, int max_step, int logits_seq_len,
               hipStream_t s, const int8_t* logits, const T* bias, int* ids, int vocab, int k,
               float p, int* unfinished, void* state, int eos_id, float scale) {
  const std::string w(who);
  if (!logits || !bias || !ids || !unfinished || rows <= 0 || cur_len <= 0 ||
      cur_len >= max_step || logits_seq_len <= 0 || vocab <= 0)
    return lsh_fail(LSH_ERR_INVALID, (w + ": bad arguments").c_str());
  if (k != 1 && (!state || (reinterpret_cast<uintptr_t>(state) & 15u) != 0))
    return lsh_fail(LSH_ERR_INVALID,
                    (w + ": random sampling needs the generator state array (lsh_rng_setup)").c_str());
  if (vocab > (1 << kSampleIdBits))
    return lsh_fail(LSH_ERR_UNSUPPORTED, (w + ": vocabulary above 2^20 ids").c_str());
  dec_sample_kernel<T><<<rows, kSampleThreads, 0, s>>>(logits, bias, ids, vocab, max_step, cur_len,
                                                       logits_seq_len, unfinished, eos_id, k, p,
                                                       scale, static_cast<SampleState*>(state));
  return lsh_check_launch("dec_sample_kernel");
}

}  // namespace

template <typename T>
int dec_topk_sample_i8I(int batch_size, int batch_seq_len, int max_step, int logits_seq_len,
                        hipStream_t s, const int8_t* logits, const T* logit_bias, int* ids,
                        int vocab_size, int k, int* unfinished, void* state, int eos_id,
                        float dequant_scale) {
  if (k != 1 && k != 2 && k != 4 && k != 8 && k != 16 && k != 32)
    return lsh_fail(LSH_ERR_INVALID, "topk argument should be in [1,2,4,8,16,32]");
  return dec_sample<T>("ker_topk_sample_i8I", batch_size, batch_seq_len, max_step, logits_seq_len,
                       s, logits, logit_bias, ids, vocab_size, k, 0.f, unfinished, state, eos_id,
                       dequant_scale);
}

template <typename T>
int dec_topp_sample_i8I(int batch_size, int batch_seq_len, int max_step, int logits_seq_len,
                        hipStream_t s, const int8_t* logits, const T* logit_bias, int* ids,
                        int vocab_size, float p, int* unfinished, void* state, int eos_id,
                        float dequant_scale) {
  if (!(p > 0.f) || p > 1.f)
    return lsh_fail(LSH_ERR_INVALID, "ker_topp_sample_i8I: topp outside (0, 1]");
  return dec_sample<T>("ker_topp_sample_i8I", batch_size, batch_seq_len, max_step, logits_seq_len,
                       s, logits, logit_bias, ids, vocab_size, 0, p, unfinished, state, eos_id,
                       dequant_scale);
}

#define LSH_INST(T)                                                                              \
  template int dec_topk_sample_i8I<T>(int, int, int, int, hipStream_t, const int8_t*, const T*,  \
                                      int*, int, int, int*, void*, int, float);                  \
  template int dec_topp_sample_i8I<T>(int, int, int, int, hipStream_t, const int8_t*, const T*,  \
                                      int*, int, float, int*, void*, int, float);
LSH_INST(float)
LSH_INST(__half)
#undef LSH_INST

}  // namespace lsh
