// Encoder self-attention core for the int8 layer path (fp16 attention, as in the
// reference): a stand-alone masked softmax with the reference's launcher
// signature, and a fused QK^T -> mask -> softmax -> PV kernel on fp16 MFMA that
// keeps the reference's rounding points (scores and probabilities are rounded to
// fp16 exactly where the reference stores them) without materialising the
// [B,h,S,S] score tensor in HBM.
//
// Replaces inference/model/quant_bert_encoder.cc.cu:321-347 (two cuBLAS strided
// batched GEMMs + ker_correlation_softmax_encself + ker_arrange_atten_output_i8O)
// and inference/kernels/transformerKernels.cc.cu:1119-1172.
#include <type_traits>

#include "ls_device.h"
#include "ls_launch.h"
#include "tile_common.h"

namespace lsh {

// ---------------------------------------------------------------------------------
// masked softmax over the last dim of [B, h, S, S]; one wavefront per row.
template <typename T, int ITER>
__global__ void __launch_bounds__(256)
softmax_encself_kernel(T* corr, const int* __restrict__ pad_mask, long rows, int seq_len,
                       int head_num) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int b = (int)(row / ((long)head_num * seq_len));
  const int qpos = (int)(row % seq_len);
  const int* mask = pad_mask + (long)b * seq_len;
  T* p = corr + row * seq_len;
  if (mask[qpos]) {  // padded query: the whole row is zeroed
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      int j = it * 64 + lane;
      if (j < seq_len) TT<T>::st(p, j, 0.f);
    }
    return;
  }
  float val[ITER];
  bool dead[ITER];
  float mx = kFloatInfNeg;
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    int j = it * 64 + lane;
    dead[it] = j >= seq_len || mask[j] != 0;
    val[it] = j < seq_len ? TT<T>::ld(p, j) : kFloatInfNeg;
    mx = fmaxf(mx, dead[it] ? kFloatInfNeg : val[it]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    val[it] = dead[it] ? 0.f : __expf(val[it] - mx);
    sum += val[it];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int it = 0; it < ITER; ++it) {
    int j = it * 64 + lane;
    if (j < seq_len) TT<T>::st(p, j, val[it] / sum);
  }
}

template <typename T>
int correlation_softmax_encself(int batch_size, int batch_seq_len, int head_num, hipStream_t s,
                                T* correlation, const int* src_padding_mask) {
  if (batch_size <= 0 || batch_seq_len <= 0 || head_num <= 0 || !correlation ||
      !src_padding_mask)
    return lsh_fail(LSH_ERR_INVALID, "ker_correlation_softmax_encself: bad arguments");
  if (batch_seq_len > 1024)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "ker_correlation_softmax_encself: seq_len > 1024");
  const long rows = (long)batch_size * head_num * batch_seq_len;
  const int grid = (int)((rows + 3) / 4);
#define LSH_SM_CASE(IT)                                               \
  softmax_encself_kernel<T, IT><<<grid, 256, 0, s>>>(correlation, src_padding_mask, rows, \
                                                     batch_seq_len, head_num)
  const int iters = (batch_seq_len + 63) / 64;
  if (iters <= 1) LSH_SM_CASE(1);
  else if (iters <= 2) LSH_SM_CASE(2);
  else if (iters <= 4) LSH_SM_CASE(4);
  else if (iters <= 8) LSH_SM_CASE(8);
  else LSH_SM_CASE(16);
#undef LSH_SM_CASE
  return lsh_check_launch("softmax_encself_kernel");
}

template int correlation_softmax_encself<float>(int, int, int, hipStream_t, float*, const int*);
template int correlation_softmax_encself<__half>(int, int, int, hipStream_t, __half*, const int*);

// ---------------------------------------------------------------------------------
// Fused encoder attention.
//
// Grid (ceil(S / (32 NW)), B*h), NW wavefronts (2 or 4), 32 queries per wavefront.
// Keys are processed in blocks of 128: K block row-major and V block transposed
// are staged in LDS.  Scores are computed transposed (S^T = K Q^T) with
// v_mfma_f32_32x32x16_f16 so that one lane owns one query: the row max / sum need
// a single cross-lane exchange, and the probability registers feed the P V MFMA
// directly as its B operand (the MFMA contraction slots are mapped onto the keys a
// lane already holds).  Two passes over the key blocks (max+sum, then P V); with a
// single key block (S <= 128) the scores stay in registers between the passes.
// MODE 1 turns the kernel into the causal prompt attention of the int8 GPT path
// (inference/model/quant_gpt_encoder.cc.cu:498-523 with
// inference/kernels/gptKernels_int8.cc.cu:192-222): q and k hold int8 codes as fp16
// values, so the fp32 MFMA accumulators are the exact int32 scores; a score becomes
// float(acc) * alpha * dq * dq without fp16 rounding, key j is visible to query i when
// j <= i, `pad_mask` is the per-sequence real length and queries at or beyond it give
// zeros.  Key blocks entirely to the right of the query block are skipped.
//
// MODE 2 is the attention core of the csrc encoder layer
// (csrc/layers/transformer_encoder_layer.cpp:121-135 with
// csrc/kernels/cuda/softmax_kernels.cu:35-279): `pad_mask` points to the layer's additive
// T=half mask [batch, S] (0 for tokens, a large negative value for padding), no query row
// is zeroed, a non-zero `dq` masks future keys, and the context is written with the heads
// merged, fp16 [batch, S, head_num * D].
//
// MODE 3 is MODE 0 reading the int8 output of the QKV product directly
// (inference/model/quant_bert_encoder.cc.cu:305-319 leaves it as [tokens, 3 * hidden]
// codes; ker_arrange_encself_qkv_i8I, transformerKernels_int8.cc.cu:1119-1172, turns
// them into fp16 q, k, v): `q` points to the codes, `k` to the fp16 bias [3 * hidden],
// `dq` is the dequantisation scale, and every element becomes
// half(half(code * dq) + bias) while it is staged, which is what the arrange kernel
// would have stored.  The fp16 q, k, v tensors are never written.
constexpr int kAttnEnc = 0, kAttnGpt = 1, kAttnLayer = 2, kAttnEncI8 = 3;

// ONE: the sequence fits one block of 128 keys; the multi-block paths are not compiled.
template <int D, int MODE, int NW, bool ONE>
// Two workgroups of four wavefronts share a compute unit for head sizes up to 64 (the
// compiler is told to stay within that register budget); 128 needs the whole file.
__global__ void __launch_bounds__(64 * NW, D <= 64 ? 2 : 1)
encself_attn_kernel(const __half* __restrict__ q, const __half* __restrict__ k,
                    const __half* __restrict__ v, const int* __restrict__ pad_mask,
                    __half* __restrict__ ctx, int8_t* __restrict__ ctx_q, float quant_scale, int S,
                    int head_num, float alpha, float dq, int key_len) {
  // number of keys: the layer mode (MODE 2) may attend over another sequence (cross
  // attention, cached decoding); everywhere else keys and queries are the same S positions
  const int Sk = MODE == kAttnLayer ? key_len : S;
  constexpr int KSTR = attn_kstr(D);  // halfs per K row in LDS (pad kills bank conflicts)
  constexpr int VSTR = kAttnVstr;     // halfs per V^T row in LDS
  constexpr int CH = D / 8;      // 16-byte chunks per row
  __shared__ __align__(16) _Float16 Ks[128 * KSTR];
  __shared__ __align__(16) _Float16 Vt[D * VSTR];
  __shared__ int msk[128];
  __shared__ float addm[MODE == kAttnLayer ? 128 : 1];
  constexpr bool GPT = MODE == kAttnGpt;
  const bool causal = GPT || (MODE == kAttnLayer && dq != 0.f);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int bh = blockIdx.y;
  const int b = bh / head_num, head = bh % head_num;
  constexpr int NT = 64 * NW;  // threads; 32 queries per wavefront
  const int qi = blockIdx.x * (32 * NW) + wave * 32 + l32;
  const _Float16* qb = reinterpret_cast<const _Float16*>(q) + (long)bh * S * D;
  const _Float16* kbase = reinterpret_cast<const _Float16*>(k) + (long)bh * Sk * D;
  const _Float16* vbase = reinterpret_cast<const _Float16*>(v) + (long)bh * Sk * D;

  // MODE 3: int8 codes [tokens, 3 * hidden] and the fp16 bias [3 * hidden]
  const int hidden3 = 3 * head_num * D;
  const int8_t* codes = reinterpret_cast<const int8_t*>(q) + (long)b * S * hidden3 + head * D;
  const _Float16* bias = reinterpret_cast<const _Float16*>(k) + head * D;

  v8h qreg[D / 16];
  // FAST (int8 QKV, at most 128 keys): every byte the workgroup reads -- query, key and value
  // codes, padding mask -- is requested before any of it is converted, so the kernel waits
  // for memory once; the padding mask is kept as two 64-bit words in scalar registers.
  constexpr bool FAST = ONE && MODE == kAttnEncI8;
  if constexpr (FAST) {
    constexpr int C16 = D / 16, KCH = 128 * C16 / NT;  // 16-code key chunks per thread
    constexpr int CH8 = D / 8, NP = 32 * CH8;          // value patches of 4 keys x 8 dims
    constexpr int VP = (NP + NT - 1) / NT;
    static_assert(128 * C16 % NT == 0, "key chunks must divide evenly over the threads");
    const int hid = head_num * D;
    uint4 wq[D / 32], wk[KCH];
    uint2 wv[VP][4];
    // rows past the end read the last row instead (an unconditional load; a conditional one
    // would become a branch with its own wait) and are zeroed when they are converted
#pragma unroll
    for (int kp = 0; kp < D / 32; ++kp)
      wq[kp] = *reinterpret_cast<const uint4*>(codes + (long)min(qi, S - 1) * hidden3 + kp * 32 +
                                               g * 16);
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + i * NT, row = c / C16, ch = c % C16;
      wk[i] = *reinterpret_cast<const uint4*>(codes + (long)min(row, S - 1) * hidden3 + hid +
                                              ch * 16);
    }
#pragma unroll
    for (int i = 0; i < VP; ++i) {
      const int pidx = min(tid + i * NT, NP - 1), kg = pidx / CH8, ch = pidx % CH8;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        wv[i][r] = *reinterpret_cast<const uint2*>(codes + (long)min(kg * 4 + r, S - 1) * hidden3 +
                                                   2 * hid + ch * 8);
    }
    const int pm0 = pad_mask[(long)b * S + min(lane, S - 1)];
    const int pm1 = pad_mask[(long)b * S + min(lane + 64, S - 1)];
    __builtin_amdgcn_sched_barrier(0);
    // queries: lane half g converts chunk kp * 32 + g * 16 .. + 16, then the halves swap their
    // second part (see the general path below)
#pragma unroll
    for (int kp = 0; kp < D / 32; ++kp) {
      v8h lo, hi;
      dequant16_bias(wq[kp], bias + kp * 32 + g * 16, dq, lo, hi);
      if (qi >= S) lo = hi = (v8h)(_Float16)0;
      v8h give = g == 0 ? hi : lo, take;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int t = __shfl_xor(reinterpret_cast<const int*>(&give)[j], 32, 64);
        reinterpret_cast<int*>(&take)[j] = t;
      }
      qreg[2 * kp] = g == 0 ? lo : take;
      qreg[2 * kp + 1] = g == 0 ? take : hi;
    }
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + i * NT, row = c / C16, ch = c % C16;
      v8h lo, hi;
      dequant16_bias(wk[i], bias + hid + ch * 16, dq, lo, hi);
      if (row >= S) lo = hi = (v8h)(_Float16)0;
      *reinterpret_cast<v8h*>(&Ks[row * KSTR + ch * 16]) = lo;
      *reinterpret_cast<v8h*>(&Ks[row * KSTR + ch * 16 + 8]) = hi;
    }
#pragma unroll
    for (int i = 0; i < VP; ++i) {
      const int pidx = tid + i * NT, kg = pidx / CH8, ch = pidx % CH8;
      if (pidx < NP) {
        v8h x[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          x[r] = dequant8_bias(wv[i][r], bias + 2 * hid + ch * 8, dq);
          if (kg * 4 + r >= S) x[r] = (v8h)(_Float16)0;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e)
          *reinterpret_cast<v4h*>(&Vt[(ch * 8 + e) * VSTR + kg * 4]) =
              (v4h){x[0][e], x[1][e], x[2][e], x[3][e]};
      }
    }
    const bool padk0 = pm0 != 0 || lane >= S, padk1 = pm1 != 0 || lane + 64 >= S;
    // the padding flag of this lane's query (queries and keys are the same positions)
    const uint64_t pad_q = __ballot(wave < 2 ? padk0 : padk1);
    const bool q_pad = qi >= S || ((pad_q >> ((wave & 1) * 32 + l32)) & 1) != 0;
    __syncthreads();
    const long tok = (long)b * S + qi;
    attend_block128<D>(Ks, Vt, qreg, padk0, padk1, q_pad, qi < S, alpha, quant_scale,
                       ctx ? ctx + ((long)bh * S + qi) * D : nullptr,
                       ctx_q ? ctx_q + tok * (head_num * D) + head * D : nullptr, l32, g);
    return;
  } else if (MODE == kAttnEncI8) {
#pragma unroll
    for (int kp = 0; kp < D / 32; ++kp) {
      // lane half g converts chunk kp * 32 + g * 16 .. + 16, then the halves swap their
      // second part so that lane (l32, g) ends with d = ks * 16 + g * 8 .. + 8 for both ks
      v8h lo = (v8h)(_Float16)0, hi = (v8h)(_Float16)0;
      if (qi < S) {
        const uint4 w =
            *reinterpret_cast<const uint4*>(codes + (long)qi * hidden3 + kp * 32 + g * 16);
        dequant16_bias(w, bias + kp * 32 + g * 16, dq, lo, hi);
      }
      // lane g=0 holds d 0..15 of this 32-block, lane g=1 holds d 16..31
      v8h give = g == 0 ? hi : lo, take;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int t = __shfl_xor(reinterpret_cast<const int*>(&give)[j], 32, 64);
        reinterpret_cast<int*>(&take)[j] = t;
      }
      qreg[2 * kp] = g == 0 ? lo : take;      // d = kp*32 + g*8 .. + 8
      qreg[2 * kp + 1] = g == 0 ? take : hi;  // d = kp*32 + 16 + g*8 .. + 8
    }
  } else {
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      if (qi < S)
        qreg[ks] = *reinterpret_cast<const v8h*>(qb + (long)qi * D + ks * 16 + g * 8);
      else
        qreg[ks] = (v8h)(_Float16)0;
    }
  }
  const bool q_pad = qi >= S || (MODE == kAttnLayer ? false
                                 : GPT              ? qi >= pad_mask[b]
                                                    : pad_mask[(long)b * S + qi] != 0);

  float m = kFloatInfNeg, sum = 0.f;
  v16f sc[4];
  v16f acc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;

  int nkb = ONE ? 1 : (Sk + 127) / 128;
  if (!ONE && causal) nkb = min(nkb, min((int)(blockIdx.x + 1) * (32 * NW) - 1, Sk - 1) / 128 + 1);
  if (ONE) nkb = 1;  // (a constant for the compiler)
  for (int phase = 0; phase < 2; ++phase) {
    for (int kb = 0; kb < nkb; ++kb) {
      const int key0 = kb * 128;
      const bool fresh = !(nkb == 1 && phase == 1);
      if (fresh) {
        __syncthreads();
        const bool want_v = phase == 1 || nkb == 1;
        if (MODE == kAttnEncI8) {
          constexpr int C16 = D / 16;  // 16-code chunks per row
          const int hid = head_num * D;
          for (int c = tid; c < 128 * C16; c += NT) {
            const int row = c / C16, ch = c % C16;
            v8h lo = (v8h)(_Float16)0, hi = (v8h)(_Float16)0;
            if (key0 + row < S) {
              const uint4 w = *reinterpret_cast<const uint4*>(
                  codes + (long)(key0 + row) * hidden3 + hid + ch * 16);
              dequant16_bias(w, bias + hid + ch * 16, dq, lo, hi);
            }
            *reinterpret_cast<v8h*>(&Ks[row * KSTR + ch * 16]) = lo;
            *reinterpret_cast<v8h*>(&Ks[row * KSTR + ch * 16 + 8]) = hi;
          }
          if (want_v) {
            // a lane transposes a patch of 4 keys x 16 dims: 16 stores of 4 keys each
            for (int p = tid; p < 32 * C16; p += NT) {
              const int kg = p / C16, ch = p % C16;
              v8h lo[4], hi[4];
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                lo[r] = (v8h)(_Float16)0;
                hi[r] = (v8h)(_Float16)0;
                const int key = key0 + kg * 4 + r;
                if (key < S) {
                  const uint4 w = *reinterpret_cast<const uint4*>(
                      codes + (long)key * hidden3 + 2 * hid + ch * 16);
                  dequant16_bias(w, bias + 2 * hid + ch * 16, dq, lo[r], hi[r]);
                }
              }
#pragma unroll
              for (int i = 0; i < 8; ++i) {
                *reinterpret_cast<v4h*>(&Vt[(ch * 16 + i) * VSTR + kg * 4]) =
                    (v4h){lo[0][i], lo[1][i], lo[2][i], lo[3][i]};
                *reinterpret_cast<v4h*>(&Vt[(ch * 16 + 8 + i) * VSTR + kg * 4]) =
                    (v4h){hi[0][i], hi[1][i], hi[2][i], hi[3][i]};
              }
            }
          }
        } else {
          for (int c = tid; c < 128 * CH; c += NT) {
            const int row = c / CH, ch = c % CH;
            v8h kv = (v8h)(_Float16)0;
            if (key0 + row < Sk)
              kv = *reinterpret_cast<const v8h*>(kbase + (long)(key0 + row) * D + ch * 8);
            *reinterpret_cast<v8h*>(&Ks[row * KSTR + ch * 8]) = kv;
          }
          if (want_v) {
            // a lane transposes a patch of 4 keys x 8 dims: 8 stores of 4 keys each
            for (int p = tid; p < 32 * CH; p += NT) {
              const int kg = p / CH, ch = p % CH;
              v8h vv[4];
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int key = key0 + kg * 4 + r;
                vv[r] = key < Sk ? *reinterpret_cast<const v8h*>(vbase + (long)key * D + ch * 8)
                                : (v8h)(_Float16)0;
              }
#pragma unroll
              for (int i = 0; i < 8; ++i)
                *reinterpret_cast<v4h*>(&Vt[(ch * 8 + i) * VSTR + kg * 4]) =
                    (v4h){vv[0][i], vv[1][i], vv[2][i], vv[3][i]};
            }
          }
        }
        if (tid < 128) {
          if (MODE == kAttnLayer) {
            msk[tid] = (key0 + tid < Sk) ? 0 : 1;
            addm[tid] = (key0 + tid < Sk && pad_mask != nullptr)
                            ? __half2float(reinterpret_cast<const __half*>(
                                  pad_mask)[(long)b * Sk + key0 + tid])
                            : 0.f;
          } else if (GPT) {
            msk[tid] = (key0 + tid < S) ? 0 : 1;
          } else {
            msk[tid] = (key0 + tid < S) ? pad_mask[(long)b * S + key0 + tid] : 1;
          }
        }
        __syncthreads();
#pragma unroll
        for (int sb = 0; sb < 4; ++sb) {
          v16f c;
#pragma unroll
          for (int i = 0; i < 16; ++i) c[i] = 0.f;
#pragma unroll
          for (int ks = 0; ks < D / 16; ++ks) {
            v8h a = *reinterpret_cast<const v8h*>(&Ks[(sb * 32 + l32) * KSTR + ks * 16 + g * 8]);
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qreg[ks], c, 0, 0, 0);
          }
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key_local = sb * 32 + 8 * (i / 4) + 4 * g + (i % 4);
            if (MODE == kAttnLayer) {
              float t = round_h(alpha * c[i]) + addm[key_local];
              if (msk[key_local] || (causal && key0 + key_local > qi) || !(t > 0.5f * kFloatInfNeg))
                t = kFloatInfNeg;
              sc[sb][i] = t;
            } else if (GPT) {
              sc[sb][i] = (msk[key_local] || key0 + key_local > qi) ? kFloatInfNeg
                                                                    : c[i] * alpha * dq * dq;
            } else {
              sc[sb][i] = msk[key_local] ? kFloatInfNeg : round_h(alpha * c[i]);
            }
          }
        }
      }
      if (phase == 0) {
        float bm = kFloatInfNeg;
#pragma unroll
        for (int sb = 0; sb < 4; ++sb)
#pragma unroll
          for (int i = 0; i < 16; ++i) bm = fmaxf(bm, sc[sb][i]);
        bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
        const float m_new = fmaxf(m, bm);
        const float mref = m_new == kFloatInfNeg ? 0.f : m_new;
        float part = 0.f;
        if (nkb == 1) {  // single key block: the second pass reuses the exponentials
          const float nm = -mref * 1.44269504088896340736f;
#pragma unroll
          for (int sb = 0; sb < 4; ++sb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              // one key block: exp(s - m) as 2^(s * log2(e) - m * log2(e)), one multiply-add
              sc[sb][i] = ONE ? __builtin_amdgcn_exp2f(
                                     fmaf(sc[sb][i], 1.44269504088896340736f, nm))
                               : __expf(sc[sb][i] - mref);
              part += sc[sb][i];
            }
        } else {
#pragma unroll
          for (int sb = 0; sb < 4; ++sb)
#pragma unroll
            for (int i = 0; i < 16; ++i) part += __expf(sc[sb][i] - mref);
        }
        part += __shfl_xor(part, 32, 64);
        sum = sum * __expf(m - m_new) + part;
        m = m_new;
      } else {
        // exp / sum is the correctly rounded quotient, as the reference's division gives:
        // exp * (1 / sum) differs from it by one unit in the last place often enough to flip
        // fp16 probabilities, and a deep stack amplifies such flips.  The quotient is formed
        // by the sequence the compiler emits for a float division (refined reciprocal, two
        // residual corrections) with the reciprocal taken once per query and without the
        // range scaling, which only acts on quotients far below the smallest fp16 value.
        float rs = __builtin_amdgcn_rcpf(sum);
        rs = sum > 0.f ? fmaf(fmaf(-sum, rs, 1.f), rs, rs) : 0.f;  // no visible key: all zero
        const float mref = m == kFloatInfNeg ? 0.f : m;
        // one instance per case, chosen by a uniform branch, so that neither evaluates the
        // other's exponentials
        auto pv_pass = [&](auto reuse_tag) {
        constexpr bool REUSE = decltype(reuse_tag)::value;
#pragma unroll
        for (int sb = 0; sb < 4; ++sb) {
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            v8h pb;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float s = sc[sb][8 * t + j];
              const float e = REUSE ? s : __expf(s - mref);
              float qt = e * rs;
              qt = fmaf(fmaf(-sum, qt, e), rs, qt);
              // one key block keeps one correction: with the refined reciprocal the first one
              // already lands on the correctly rounded quotient except within 2^-22 of a
              // rounding boundary of the float quotient
              if constexpr (!ONE) qt = fmaf(fmaf(-sum, qt, e), rs, qt);
              // keep the float quotient a value of its own: folded into the last correction,
              // the conversion to fp16 would round once instead of twice
              asm volatile("" : "+v"(qt));
              pb[j] = (_Float16)qt;
            }
#pragma unroll
            for (int db = 0; db < D / 32; ++db) {
              const _Float16* vrow = &Vt[(db * 32 + l32) * VSTR + sb * 32 + 16 * t + 4 * g];
              v4h lo = *reinterpret_cast<const v4h*>(vrow);
              v4h hi = *reinterpret_cast<const v4h*>(vrow + 8);
              v8h a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
              acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb, acc[db], 0, 0, 0);
            }
          }
        }
        };
        if (nkb == 1)
          pv_pass(std::true_type{});
        else
          pv_pass(std::false_type{});
      }
    }
  }

  if (qi >= S) return;
  const long tok = (long)b * S + qi;
  const int hidden = head_num * D;
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
#pragma unroll
    for (int vg = 0; vg < 4; ++vg) {
      const int dd = db * 32 + 8 * vg + 4 * g;
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = round_h(acc[db][4 * vg + j]);
      if (ctx != nullptr) {
        half4_t t;
#pragma unroll
        for (int j = 0; j < 4; ++j) t.v[j] = __float2half_rn(q_pad ? 0.f : o[j]);
        if (MODE == kAttnLayer)
          *reinterpret_cast<half4_t*>(ctx + tok * hidden + head * D + dd) = t;
        else
          *reinterpret_cast<half4_t*>(ctx + ((long)bh * S + qi) * D + dd) = t;
      }
      if (ctx_q != nullptr) {
        // a padded query gives zeros, whose code is 0
        const uint32_t w4 = float2int8_pack4(o[0], o[1], o[2], o[3], quant_scale);
        *reinterpret_cast<uint32_t*>(ctx_q + tok * hidden + head * D + dd) = q_pad ? 0u : w4;
      }
    }
  }
}

// 4 wavefronts (128 queries) per workgroup once a sequence has more than 64 queries, so
// that a (batch, head) pair with up to 128 keys is staged once; 2 wavefronts otherwise.
template <int MODE>
static bool launch_attn(int dim_per_head, int seq_len, int batch_heads, hipStream_t s,
                        const __half* q, const __half* k, const __half* v, const int* pad_mask,
                        __half* ctx, int8_t* ctx_q, float quant_scale, int head_num, float alpha,
                        float dq, int key_len = -1) {
  if (key_len < 0) key_len = seq_len;  // self attention: as many keys as queries
#define LSH_ATTN(DD, NWV)                                                                      \
  if (key_len <= 128)                                                                          \
    encself_attn_kernel<DD, MODE, NWV, true>                                                   \
        <<<dim3((seq_len + 32 * NWV - 1) / (32 * NWV), batch_heads), 64 * NWV, 0, s>>>(        \
            q, k, v, pad_mask, ctx, ctx_q, quant_scale, seq_len, head_num, alpha, dq, key_len); \
  else                                                                                         \
    encself_attn_kernel<DD, MODE, NWV, false>                                                  \
      <<<dim3((seq_len + 32 * NWV - 1) / (32 * NWV), batch_heads), 64 * NWV, 0, s>>>(          \
          q, k, v, pad_mask, ctx, ctx_q, quant_scale, seq_len, head_num, alpha, dq, key_len)
  const bool wide = seq_len > 64;
  switch (dim_per_head) {
    case 32:
      if (wide) { LSH_ATTN(32, 4); } else { LSH_ATTN(32, 2); }
      return true;
    case 64:
      if (wide) { LSH_ATTN(64, 4); } else { LSH_ATTN(64, 2); }
      return true;
    case 128:
      if (wide) { LSH_ATTN(128, 4); } else { LSH_ATTN(128, 2); }
      return true;
    default:
      return false;
  }
#undef LSH_ATTN
}

int encself_attention_f16(const __half* q, const __half* k, const __half* v, const int* pad_mask,
                          __half* ctx, int8_t* ctx_q, float quant_scale, int batch, int seq_len,
                          int head_num, int dim_per_head, hipStream_t s) {
  if (batch <= 0 || seq_len <= 0 || head_num <= 0 || !q || !k || !v || !pad_mask ||
      (!ctx && !ctx_q))
    return lsh_fail(LSH_ERR_INVALID, "encself_attention: bad arguments");
  if (seq_len > 1024) return lsh_fail(LSH_ERR_UNSUPPORTED, "encself_attention: seq_len > 1024");
  if (((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
        reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(ctx) |
        reinterpret_cast<uintptr_t>(ctx_q)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "encself_attention: pointers must be 16-byte aligned");
  const float alpha = __half2float(__float2half_rn(sqrtf(1.f / (float)dim_per_head)));
  if (!launch_attn<kAttnEnc>(dim_per_head, seq_len, batch * head_num, s, q, k, v, pad_mask, ctx,
                             ctx_q, quant_scale, head_num, alpha, 0.f))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "encself_attention: dim_per_head must be 32, 64 or 128");
  return lsh_check_launch("encself_attn_kernel");
}

// The same attention reading the int8 output of the QKV product [batch * seq_len,
// 3 * hidden] and the fp16 bias [3 * hidden] (MODE 3 above).
int encself_attention_i8qkv(const int8_t* qkv, const __half* qkv_bias, float dequant_scale,
                            const int* pad_mask, __half* ctx, int8_t* ctx_q, float quant_scale,
                            int batch, int seq_len, int head_num, int dim_per_head, hipStream_t s) {
  if (batch <= 0 || seq_len <= 0 || head_num <= 0 || !qkv || !qkv_bias || !pad_mask ||
      (!ctx && !ctx_q))
    return lsh_fail(LSH_ERR_INVALID, "encself_attention_i8qkv: bad arguments");
  if (seq_len > 1024)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "encself_attention_i8qkv: seq_len > 1024");
  if (((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(qkv_bias) |
        reinterpret_cast<uintptr_t>(ctx) | reinterpret_cast<uintptr_t>(ctx_q)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "encself_attention_i8qkv: pointers must be 16-byte aligned");
  const float alpha = __half2float(__float2half_rn(sqrtf(1.f / (float)dim_per_head)));
  const __half* q = reinterpret_cast<const __half*>(qkv);
  if (!launch_attn<kAttnEncI8>(dim_per_head, seq_len, batch * head_num, s, q, qkv_bias, nullptr,
                               pad_mask, ctx, ctx_q, quant_scale, head_num, alpha, dequant_scale))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                        "encself_attention_i8qkv: dim_per_head must be 32, 64 or 128");
  return lsh_check_launch("encself_attn_kernel<i8 qkv>");
}

int gpt_prefill_attention_f16(const __half* q_codes, const __half* k_codes, const __half* v,
                              const int* real_seq_len, __half* ctx, int8_t* ctx_q,
                              float quant_scale, float dequant_scale, int batch, int seq_len,
                              int head_num, int dim_per_head, hipStream_t s) {
  if (batch <= 0 || seq_len <= 0 || head_num <= 0 || !q_codes || !k_codes || !v ||
      !real_seq_len || (!ctx && !ctx_q))
    return lsh_fail(LSH_ERR_INVALID, "gpt_prefill_attention: bad arguments");
  if (seq_len > 4096)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "gpt_prefill_attention: seq_len > 4096");
  if (((reinterpret_cast<uintptr_t>(q_codes) | reinterpret_cast<uintptr_t>(k_codes) |
        reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(ctx) |
        reinterpret_cast<uintptr_t>(ctx_q)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "gpt_prefill_attention: pointers must be 16-byte aligned");
  const float alpha = __half2float(__float2half_rn(sqrtf(1.f / (float)dim_per_head)));
  if (!launch_attn<kAttnGpt>(dim_per_head, seq_len, batch * head_num, s, q_codes, k_codes, v,
                             real_seq_len, ctx, ctx_q, quant_scale, head_num, alpha,
                             dequant_scale))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                        "gpt_prefill_attention: dim_per_head must be 32, 64 or 128");
  return lsh_check_launch("encself_attn_kernel<GPT>");
}

// Attention core of the csrc encoder layer: q, k, v fp16 [batch, heads, S, D], additive
// fp16 mask [batch, S] (may be null), context fp16 [batch, S, heads * D].
int layer_attention_f16(const __half* q, const __half* k, const __half* v, const __half* add_mask,
                        __half* ctx, int batch, int seq_len, int head_num, int dim_per_head,
                        bool mask_future, hipStream_t s) {
  return layer_cross_attention_f16(q, k, v, add_mask, ctx, batch, seq_len, seq_len, head_num,
                                   dim_per_head, mask_future, s);
}

// The same with its own number of keys: q [batch, heads, q_len, D], k and v [batch, heads,
// k_len, D], additive mask [batch, k_len] (may be null), context [batch, q_len, heads * D].
// The decoder layer of the csrc tree uses it for the cross attention (k_len = source length;
// csrc/layers/transformer_decoder_layer.cpp:333-357) and for a cached step (q_len = 1,
// k_len = step + 1, :173-189).  mask_future needs q_len == k_len.
int layer_cross_attention_f16(const __half* q, const __half* k, const __half* v,
                              const __half* add_mask, __half* ctx, int batch, int seq_len,
                              int key_len, int head_num, int dim_per_head, bool mask_future,
                              hipStream_t s) {
  if (batch <= 0 || seq_len <= 0 || key_len <= 0 || head_num <= 0 || !q || !k || !v || !ctx ||
      (mask_future && seq_len != key_len))
    return lsh_fail(LSH_ERR_INVALID, "layer_attention: bad arguments");
  if (seq_len > 1024 || key_len > 1024)
    return lsh_fail(LSH_ERR_UNSUPPORTED, "layer_attention: seq_len > 1024");
  if (((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
        reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(ctx)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "layer_attention: pointers must be 16-byte aligned");
  // strided_batch_gemm alpha: T(1.0) / T(sqrt(d)) (transformer_encoder_layer.cpp:48-50)
  const float alpha = __half2float(
      __float2half_rn(1.0f / __half2float(__float2half_rn(sqrtf((float)dim_per_head)))));
  const int* m = reinterpret_cast<const int*>(add_mask);
  const float causal = mask_future ? 1.f : 0.f;
  if (!launch_attn<kAttnLayer>(dim_per_head, seq_len, batch * head_num, s, q, k, v, m, ctx,
                               nullptr, 0.f, head_num, alpha, causal, key_len))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "layer_attention: dim_per_head must be 32, 64 or 128");
  return lsh_check_launch("encself_attn_kernel<layer>");
}

}  // namespace lsh
