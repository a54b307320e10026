// Prompt pass of the int8 GPT model on int8 codes end to end
// (inference/model/quant_gpt_encoder.cc.cu:489-530):
//
//   gpt_arrange_qkv_prefill_i8   ker_arrange_encself_qkv_i8I_i8O (:489-496): dequantise the QKV
//                                product, add the bias, requantise -- q codes [batch, head, seq, d]
//                                and the k / v codes straight into the caches
//                                [batch, head, max_step, d] (nothing is written as fp16);
//   gpt_prefill_attention_i8     the int8 q.K^T GEMM (:498-505), ker_correlation_softmax_gpt_i32I
//                                (inference/kernels/gptKernels_int8.cc.cu:192-250), the P.V GEMM
//                                (:512-518) and ker_arrange_atten_output_i8O (:520-523) in one
//                                causal kernel that reads q codes and the caches.
//
// The attention kernel: heads of 64, one workgroup of 4 wavefronts per (sequence, head, block of
// 128 queries).  All the key codes the block may see (keys 0 .. its last query: 64 bytes per
// key) are brought into LDS once and serve both passes of the exact two-pass soft-max; scores are
// v_mfma_i32_32x32x32_i8 products of codes -- the int32 scores of the reference bit for bit --
// computed transposed (keys x queries), so a lane owns one query.  Values are dequantised while
// they are staged (half(code / quant_scale), what the arrange kernel of the reference stores,
// through a 256-entry table) into a transposed fp16 tile, two tiles alternating, the next block's
// codes requested before the current block is multiplied.  Only the diagonal key block needs the
// causal mask; blocks to the right of the diagonal are never touched.  Rounding points as the
// reference: probability -> fp16, context -> fp16 -> int8; the quotient exp / sum is the
// correctly rounded one (see encself_attn_kernel).  Workgroups of the last query blocks (most key
// blocks) are launched first.
#include "ls_device.h"
#include "ls_launch.h"
#include "tile_common.h"

#include <atomic>
#include <mutex>

namespace lsh {

// ---------------------------------------------------------------------------------
// A workgroup owns one 128-byte column group (128 / d heads) of one part (q, k or v) of one
// sequence and walks its tokens, 32 rows per pass, 16 codes per thread: what it writes is
// contiguous per head.
// ---------------------------------------------------------------------------------
template <int UNR>
__global__ void __launch_bounds__(256)
gpt_arrange_qkv_prefill_i8_kernel(const int8_t* __restrict__ ori, const __half* __restrict__ bias,
                                  int8_t* __restrict__ q_codes, int8_t* __restrict__ k_cache,
                                  int8_t* __restrict__ v_cache, int seq_len, int d, int head_num,
                                  int groups, int max_step, float ds, float qs) {
#pragma clang fp contract(off)
  const int hidden = d * head_num;
  const int grp = blockIdx.x % groups, which = (blockIdx.x / groups) % 3;
  const int b = blockIdx.x / (groups * 3);
  const int row = threadIdx.x >> 3, seg = threadIdx.x & 7;
  const int col = grp * 128 + seg * 16;  // first of this thread's 16 columns inside the part
  const int head = col / d, dim = col % d;
  float bv[16];
  {
    const half8_t b0 = *reinterpret_cast<const half8_t*>(bias + (long)which * hidden + col);
    const half8_t b1 = *reinterpret_cast<const half8_t*>(bias + (long)which * hidden + col + 8);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      bv[k] = __half2float(b0.v[k]);
      bv[8 + k] = __half2float(b1.v[k]);
    }
  }
  const int8_t* src = ori + ((long)b * seq_len * 3 + which) * hidden + col;
  const long bh = (long)b * head_num + head;
  int8_t* dst = which == 0   ? q_codes + bh * seq_len * d + dim
                : which == 1 ? k_cache + bh * max_step * d + dim
                             : v_cache + bh * max_step * d + dim;
  for (int s0 = row; s0 < seq_len; s0 += 32 * UNR) {
    uint4 w[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int s = min(s0 + 32 * u, seq_len - 1);
      w[u] = *reinterpret_cast<const uint4*>(src + (long)s * 3 * hidden);
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int s = s0 + 32 * u;
      if (s >= seq_len) break;
      const uint32_t wi[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
      uint32_t o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int q[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float val = (float)unpack_i8(wi[j], k) * ds + bv[4 * j + k];
          q[k] = float2int8(val, qs);
        }
        o[j] = pack4_i8(q[0], q[1], q[2], q[3]);
      }
      *reinterpret_cast<uint4*>(dst + (long)s * d) = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
}

static std::atomic<bool> g_prefill_i8_in_models{true};
bool gpt_prefill_i8_enable(bool on) {
  const bool prev = g_prefill_i8_in_models.exchange(on);
  if (prev != on) route_epoch_bump();
  return prev;
}
bool gpt_prefill_i8_enabled() { return g_prefill_i8_in_models.load(std::memory_order_relaxed); }

bool gpt_prefill_i8_supported(int seq_len, int head_num, int dim_per_head) {
  return dim_per_head == 64 && head_num > 0 && seq_len >= 1 && seq_len <= 1024;
}

int gpt_arrange_qkv_prefill_i8(int batch_token_num, int hidden_size, hipStream_t s,
                               const int8_t* ori_qkv, const __half* qkv_bias, int8_t* q_codes,
                               int8_t* k_cache, int8_t* v_cache, int batch_seq_len,
                               int dim_per_head, int head_num, int max_step, float dequant_scale,
                               float quant_scale) {
  if (!ori_qkv || !qkv_bias || !q_codes || !k_cache || !v_cache || batch_token_num <= 0 ||
      batch_seq_len <= 0 || batch_token_num % batch_seq_len != 0 || dim_per_head <= 0 ||
      hidden_size != dim_per_head * head_num || batch_seq_len > max_step)
    return lsh_fail(LSH_ERR_INVALID, "gpt_arrange_qkv_prefill_i8: bad arguments");
  if (hidden_size % 128 != 0 || dim_per_head % 16 != 0 ||
      (128 % dim_per_head != 0 && dim_per_head % 128 != 0))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "gpt_arrange_qkv_prefill_i8: hidden must be a multiple of 128 and the head "
                    "size 16, 32, 64 or a multiple of 128");
  if (((reinterpret_cast<uintptr_t>(ori_qkv) | reinterpret_cast<uintptr_t>(qkv_bias) |
        reinterpret_cast<uintptr_t>(q_codes) | reinterpret_cast<uintptr_t>(k_cache) |
        reinterpret_cast<uintptr_t>(v_cache)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "gpt_arrange_qkv_prefill_i8: pointers must be 16-byte aligned");
  const int batch = batch_token_num / batch_seq_len, groups = hidden_size / 128;
  if ((long)batch * 3 * groups >= (1L << 30))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "gpt_arrange_qkv_prefill_i8: too many workgroups");
  if (batch_seq_len > 64)
    gpt_arrange_qkv_prefill_i8_kernel<4><<<batch * 3 * groups, 256, 0, s>>>(
        ori_qkv, qkv_bias, q_codes, k_cache, v_cache, batch_seq_len, dim_per_head, head_num, groups,
        max_step, dequant_scale, quant_scale);
  else
    gpt_arrange_qkv_prefill_i8_kernel<2><<<batch * 3 * groups, 256, 0, s>>>(
        ori_qkv, qkv_bias, q_codes, k_cache, v_cache, batch_seq_len, dim_per_head, head_num, groups,
        max_step, dequant_scale, quant_scale);
  return lsh_check_launch("gpt_arrange_qkv_prefill_i8_kernel");
}

// ---------------------------------------------------------------------------------
// The attention.  LDS: key codes (nkb_max * 128 rows of 64 bytes, the four 16-byte chunks of a
// row XOR-swizzled by (row / 2) % 4 so that the fragment reads of 8 neighbouring rows hit 8
// different 16-byte slots), two transposed value tiles [64][132] fp16, the 256-entry table.
// ---------------------------------------------------------------------------------
constexpr int kPfVstr = kAttnVstr;  // halfs per V^T row
constexpr int kPfVtBytes = 64 * kPfVstr * 2;
static size_t gpt_prefill_lds_bytes(int seq_len) {
  return (size_t)((seq_len + 127) / 128) * 128 * 64 + 2 * kPfVtBytes + 512;
}

__global__ void __launch_bounds__(256, 2)
gpt_prefill_attn_i8_kernel(const int8_t* __restrict__ q_codes, const int8_t* __restrict__ k_cache,
                           const int8_t* __restrict__ v_cache, const int* __restrict__ real_seq_len,
                           int8_t* __restrict__ ctx_q, float quant_scale, float v_quant_scale,
                           int S, int head_num, int max_step, float alpha, float dq, int BH) {
  constexpr int D = 64, VSTR = kPfVstr;
  extern __shared__ __align__(16) int8_t smem[];
  const int nkb_max = (S + 127) / 128;
  int8_t* Ks = smem;
  _Float16* Vt0 = reinterpret_cast<_Float16*>(smem + (size_t)nkb_max * 128 * 64);
  _Float16* tabh = Vt0 + 2 * 64 * VSTR;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  // the query blocks with the most key blocks first
  const int qb = nkb_max - 1 - (int)(blockIdx.x / BH), bh = blockIdx.x % BH;
  const int b = bh / head_num, head = bh % head_num;
  const int nkb = qb + 1;  // key blocks 0 .. qb (causal)
  const int qi = qb * 128 + wave * 32 + l32;
  const int8_t* qbase = q_codes + (long)bh * S * D;
  const int8_t* kbase = k_cache + (long)bh * max_step * D;
  const int8_t* vbase = v_cache + (long)bh * max_step * D;

  // ---- everything the prologue reads is requested before any of it is used
  v4i qreg[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
    qreg[ks] = *reinterpret_cast<const v4i*>(qbase + (long)min(qi, S - 1) * D + ks * 32 + g * 16);
  const int real_len = real_seq_len[b];
  // value codes of a key block: a thread takes a patch of 4 keys x 8 dims
  const int vkg = tid >> 3, vch = tid & 7;
  uint2 vcur[4], vnext[4];
  auto request_v = [&](uint2 (&w)[4], int kb) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      w[r] = *reinterpret_cast<const uint2*>(
          vbase + (long)min(kb * 128 + vkg * 4 + r, S - 1) * D + vch * 8);
  };
  {
    // key codes straight into LDS (no registers in between): an instruction of a wavefront
    // fills 16 rows, lane p writing slot p % 4 of row p / 4 -- so it fetches the chunk that the
    // swizzle puts there
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)Ks);
    for (int i = wave; i < 8 * nkb; i += 4) {
      const int row = i * 16 + (lane >> 2);
      const int ch = (lane & 3) ^ ((row >> 1) & 3);
      const uint32_t voff = (uint32_t)min(row, S - 1) * D + ch * 16;
      const uint32_t lds = __builtin_amdgcn_readfirstlane(lds0 + i * 1024);
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff),
                   "s"(kbase)
                   : "memory");
    }
    request_v(vcur, 0);
    tabh[tid] = (_Float16)((float)(tid - 128) / v_quant_scale);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the key codes have landed
  }
  const bool q_pad = qi >= S || qi >= real_len;
  __syncthreads();

  // the int32 scores of one block of 32 keys against this lane's query, as floats
  auto scores32 = [&](int kb, int sb, v16f& out, bool diag) {
    v16i c = (v16i)0;
    const int row = kb * 128 + sb * 32 + l32;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const v4i a = *reinterpret_cast<const v4i*>(
          Ks + row * 64 + (((ks * 2 + g) ^ ((row >> 1) & 3)) << 4));
      c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qreg[ks], c, 0, 0, 0);
    }
    const int key0 = kb * 128 + sb * 32 + 4 * g;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float t = (float)c[i] * alpha * dq * dq;
      out[i] = (diag && key0 + 8 * (i / 4) + (i % 4) > qi) ? kFloatInfNeg : t;
    }
  };

  // ---- pass 1: maximum and sum of exponentials over all visible keys
  float m = kFloatInfNeg, sum = 0.f;
  for (int kb = 0; kb < nkb; ++kb) {
    v16f sc[4];
    if (kb == qb) {
#pragma unroll
      for (int sb = 0; sb < 4; ++sb) scores32(kb, sb, sc[sb], true);
    } else {
#pragma unroll
      for (int sb = 0; sb < 4; ++sb) scores32(kb, sb, sc[sb], false);
    }
    float bm = kFloatInfNeg;
#pragma unroll
    for (int sb = 0; sb < 4; ++sb)
#pragma unroll
      for (int i = 0; i < 16; ++i) bm = fmaxf(bm, sc[sb][i]);
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
    const float m_new = fmaxf(m, bm);
    const float mref = m_new == kFloatInfNeg ? 0.f : m_new;
    float part = 0.f;
#pragma unroll
    for (int sb = 0; sb < 4; ++sb)
#pragma unroll
      for (int i = 0; i < 16; ++i) part += __expf(sc[sb][i] - mref);
    part += __shfl_xor(part, 32, 64);
    sum = sum * __expf(m - m_new) + part;
    m = m_new;
  }

  // ---- pass 2: probabilities (fp16) times values
  v16f acc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
  float rs = __builtin_amdgcn_rcpf(sum);
  rs = sum > 0.f ? fmaf(fmaf(-sum, rs, 1.f), rs, rs) : 0.f;
  const float mref = m == kFloatInfNeg ? 0.f : m;
  for (int kb = 0; kb < nkb; ++kb) {
    _Float16* Vt = Vt0 + (kb & 1) * (64 * VSTR);
    if (kb + 1 < nkb) request_v(vnext, kb + 1);
    {
      // dequantise through the table and store the patch transposed: 8 stores of 4 keys
      v8h x[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const uint32_t u0 = vcur[r].x ^ 0x80808080u, u1 = vcur[r].y ^ 0x80808080u;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[r][e] = tabh[(u0 >> (8 * e)) & 0xff];
          x[r][4 + e] = tabh[(u1 >> (8 * e)) & 0xff];
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)
        *reinterpret_cast<v4h*>(&Vt[(vch * 8 + e) * VSTR + vkg * 4]) =
            (v4h){x[0][e], x[1][e], x[2][e], x[3][e]};
    }
    __syncthreads();
#pragma unroll
    for (int sb = 0; sb < 4; ++sb) {
      v16f sc;
      if (kb == qb) scores32(kb, sb, sc, true);
      else scores32(kb, sb, sc, false);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        v8h pb;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float e = __expf(sc[8 * t + j] - mref);
          float qt = e * rs;
          qt = fmaf(fmaf(-sum, qt, e), rs, qt);
          qt = fmaf(fmaf(-sum, qt, e), rs, qt);
          // keep the float quotient a value of its own: folded into the last correction, the
          // conversion to fp16 would round once instead of twice
          asm volatile("" : "+v"(qt));
          pb[j] = (_Float16)qt;
        }
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          const _Float16* vrow = &Vt[(db * 32 + l32) * VSTR + sb * 32 + 16 * t + 4 * g];
          const v4h lo = *reinterpret_cast<const v4h*>(vrow);
          const v4h hi = *reinterpret_cast<const v4h*>(vrow + 8);
          const v8h a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb, acc[db], 0, 0, 0);
        }
      }
    }
    if (kb + 1 < nkb) {
#pragma unroll
      for (int r = 0; r < 4; ++r) vcur[r] = vnext[r];
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
      const uint32_t w4 = float2int8_pack4(o[0], o[1], o[2], o[3], quant_scale);
      // a padded query gives zeros, whose code is 0
      *reinterpret_cast<uint32_t*>(ctx_q + tok * hidden + head * D + dd) = q_pad ? 0u : w4;
    }
  }
}

int gpt_prefill_attention_i8(const int8_t* q_codes, const int8_t* k_cache, const int8_t* v_cache,
                             const int* real_seq_len, int8_t* ctx_q, float quant_scale,
                             float dequant_scale, float v_quant_scale, int batch, int seq_len,
                             int head_num, int dim_per_head, int max_step, hipStream_t s) {
  if (batch <= 0 || seq_len <= 0 || head_num <= 0 || !q_codes || !k_cache || !v_cache ||
      !real_seq_len || !ctx_q || seq_len > max_step || !(v_quant_scale > 0.f))
    return lsh_fail(LSH_ERR_INVALID, "gpt_prefill_attention_i8: bad arguments");
  if (!gpt_prefill_i8_supported(seq_len, head_num, dim_per_head))
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "gpt_prefill_attention_i8: heads of 64 and at most 1024 tokens");
  if (((reinterpret_cast<uintptr_t>(q_codes) | reinterpret_cast<uintptr_t>(k_cache) |
        reinterpret_cast<uintptr_t>(v_cache) | reinterpret_cast<uintptr_t>(ctx_q)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "gpt_prefill_attention_i8: pointers must be 16-byte aligned");
  const long BH = (long)batch * head_num;
  const int nqb = (seq_len + 127) / 128;
  if (BH * nqb >= (1L << 30))
    return lsh_fail(LSH_ERR_UNSUPPORTED, "gpt_prefill_attention_i8: too many workgroups");
  const size_t smem = gpt_prefill_lds_bytes(1024);
  {
    // more than the default dynamic LDS limit: raise it once per device
    static std::mutex mu;
    static unsigned long long raised = 0;
    int dev = 0;
    if (lsh_check_hip(hipGetDevice(&dev), "hipGetDevice")) return LSH_ERR_HIP;
    std::lock_guard<std::mutex> lock(mu);
    if (dev >= 64 || !((raised >> dev) & 1)) {
      if (lsh_check_hip(
              hipFuncSetAttribute(reinterpret_cast<const void*>(gpt_prefill_attn_i8_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
              "hipFuncSetAttribute(gpt_prefill_attn_i8_kernel)"))
        return LSH_ERR_HIP;
      if (dev < 64) raised |= 1ull << dev;
    }
  }
  const float alpha = __half2float(__float2half_rn(sqrtf(1.f / (float)dim_per_head)));
  gpt_prefill_attn_i8_kernel<<<(int)(BH * nqb), 256, gpt_prefill_lds_bytes(seq_len), s>>>(
      q_codes, k_cache, v_cache, real_seq_len, ctx_q, quant_scale, v_quant_scale, seq_len, head_num,
      max_step, alpha, dequant_scale, (int)BH);
  return lsh_check_launch("gpt_prefill_attn_i8_kernel");
}

}  // namespace lsh
