// Operator kernels of the quantised layer path (the launch_* family of
// lightseq/csrc/kernels/cuda/includes/kernels.h), forward only.
//
// All of them are HBM-bound streaming kernels: one 16-byte load per lane for T data
// (8 halfs / 4 floats), the matching 8- or 4-byte access for int8 codes and mask bytes,
// every tensor touched once.  Clip values live in device memory (T scalars inside the
// layer's parameter blob), so no kernel needs a host copy of them.  Row kernels
// (layer norm, softmax) give one 64-lane wavefront to a row and reduce with cross-lane
// shuffles.  Dropout ratios must be 0 (inference); the mask outputs are still written.
#include "ls_device.h"
#include "ls_launch.h"

namespace lsh {

namespace {

constexpr float kQ = 127.0f;               // kernels.h:20
constexpr float kLnEps = 1e-8f;            // normalize_kernels.cu:12
constexpr float kSoftmaxEps = 1e-8f;       // softmax_kernels.cu:11

template <typename T>
struct Vec {
  static constexpr int N = sizeof(T) == 2 ? 8 : 4;
};

__device__ __forceinline__ void ldv(const float* p, long i, float (&o)[4]) { ld4(p, i, o); }
__device__ __forceinline__ void ldv(const __half* p, long i, float (&o)[8]) {
  half8_t t = *reinterpret_cast<const half8_t*>(p + i);
#pragma unroll
  for (int k = 0; k < 8; ++k) o[k] = __half2float(t.v[k]);
}
__device__ __forceinline__ void stv(float* p, long i, const float (&o)[4]) { st4(p, i, o); }
__device__ __forceinline__ void stv(__half* p, long i, const float (&o)[8]) {
  half8_t t;
#pragma unroll
  for (int k = 0; k < 8; ++k) t.v[k] = __float2half_rn(o[k]);
  *reinterpret_cast<half8_t*>(p + i) = t;
}
// N int8 codes / mask bytes at byte offset i (i % N == 0)
template <int N>
__device__ __forceinline__ void ldq(const int8_t* p, long i, int (&o)[N]) {
  if (N == 8) {
    uint2 w = *reinterpret_cast<const uint2*>(p + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      o[k] = unpack_i8(w.x, k);
      o[4 + k] = unpack_i8(w.y, k);
    }
  } else {
    uint32_t w = *reinterpret_cast<const uint32_t*>(p + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = unpack_i8(w, k);
  }
}
template <int N>
__device__ __forceinline__ void stq(int8_t* p, long i, const int (&q)[N]) {
  if (N == 8) {
    uint2 w;
    w.x = pack4_i8(q[0], q[1], q[2], q[3]);
    w.y = pack4_i8(q[4], q[5], q[6], q[7]);
    *reinterpret_cast<uint2*>(p + i) = w;
  } else {
    *reinterpret_cast<uint32_t*>(p + i) = pack4_i8(q[0], q[1], q[2], q[3]);
  }
}
// mask[i .. i+N) |= bits
template <int N>
__device__ __forceinline__ void or_mask(uint8_t* p, long i, const int (&m)[N]) {
  if (p == nullptr) return;
  if (N == 8) {
    uint2 w = *reinterpret_cast<uint2*>(p + i);
    w.x |= (uint32_t)m[0] | ((uint32_t)m[1] << 8) | ((uint32_t)m[2] << 16) | ((uint32_t)m[3] << 24);
    w.y |= (uint32_t)m[4] | ((uint32_t)m[5] << 8) | ((uint32_t)m[6] << 16) | ((uint32_t)m[7] << 24);
    *reinterpret_cast<uint2*>(p + i) = w;
  } else {
    uint32_t w = *reinterpret_cast<uint32_t*>(p + i);
    w |= (uint32_t)m[0] | ((uint32_t)m[1] << 8) | ((uint32_t)m[2] << 16) | ((uint32_t)m[3] << 24);
    *reinterpret_cast<uint32_t*>(p + i) = w;
  }
}

// kernels.h:425-435
__device__ __forceinline__ int clip_mask_bits(float v, float cmax, int bit, bool symmetry = true) {
  if (v >= cmax) return 1 << (bit - 1);
  if (symmetry && v <= -cmax) return 1 << bit;
  return 0;
}
// kernels.h:463-471
__device__ __forceinline__ int quantize_b(float x, float cmax, int& mask, int bit) {
  mask = clip_mask_bits(x, cmax, bit);
  const float scale = cmax / kQ;
  const float q = floorf(x / scale + 0.5f);
  return (int)fminf(fmaxf(q, -kQ), kQ);
}
// kernels.h:473-488
__device__ __forceinline__ float fake_quantize_b(float x, float cmax, int& mask, int bit,
                                                 bool symmetry) {
  mask = clip_mask_bits(x, cmax, bit, symmetry);
  float scale = cmax / kQ;
  if (!symmetry) scale /= 2;
  float f = x / scale;
  if (!symmetry) f -= kQ;
  float q = fminf(fmaxf(floorf(f + 0.5f), -kQ), kQ);
  return symmetry ? q * scale : (q + kQ) * scale;
}
// kernels.h:497-501
__device__ __forceinline__ float dequantize_b(int q, float cmax) {
  const float r = (float)q * (cmax / kQ);
  return fminf(fmaxf(r, -cmax), cmax);
}
// dequantise + bias as T adds them (half: rounded operand, half add)
template <typename T>
__device__ __forceinline__ float deq_bias(int q, float cmax, float bias) {
  return TT<T>::rnd(TT<T>::rnd(dequantize_b(q, cmax)) + bias);
}
template <typename T>
__device__ __forceinline__ float cm(const T* p, int i = 0) {
  return TT<T>::ld(p, i);
}

// dropout_kernels.cu:25-59: float GELU/ReLU for T=float, the half2 forms for T=half
template <typename T, int ACT>
__device__ __forceinline__ float act_b(float x) {
  if (ACT == 1) return fmaxf(x, 0.f);
  if (sizeof(T) == 2) {
    const float p3 = TT<T>::rnd(x * TT<T>::rnd(x * x));
    const float cdf = 0.5f * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * p3)));
    return TT<T>::rnd(x * TT<T>::rnd(cdf));
  }
  return gelu_tanh(x);
}

inline int grid_for(long nvec) { return (int)((nvec + 255) / 256); }

// ---------------------------------------------------------------------------------
// quantize / fake_quantize / dequantize (quantize_kernels.cu)
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
quantize_b_kernel(int8_t* __restrict__ q, uint8_t* cmask, float* __restrict__ alpha,
                  const T* __restrict__ f, const T* __restrict__ cmax, long numel,
                  int alpha_count, int bit) {
  constexpr int N = Vec<T>::N;
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * N;
  const float c = cm(cmax);
  if (alpha != nullptr) {
    const float a = c * cm(cmax, 1) / (cm(cmax, 2) * kQ);
    for (long j = (long)blockIdx.x * 256 + threadIdx.x; j < alpha_count;
         j += (long)gridDim.x * 256)
      alpha[j] = a;
  }
  if (i >= numel) return;
  float x[N];
  int qv[N], m[N];
  ldv(f, i, x);
#pragma unroll
  for (int k = 0; k < N; ++k) qv[k] = quantize_b(x[k], c, m[k], bit);
  stq<N>(q, i, qv);
  or_mask<N>(cmask, i, m);
}

template <typename T>
__global__ void __launch_bounds__(256)
fake_quantize_b_kernel(uint8_t* cmask, float* __restrict__ alpha, T* out, const T* in,
                       const T* __restrict__ cmax, long numel, int bit, int symmetry) {
  constexpr int N = Vec<T>::N;
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * N;
  const float c = cm(cmax);
  // quantize_kernels.cu:185-190: both "input" and "weight" clip are clip_max[0] here
  if (alpha != nullptr && blockIdx.x == 0 && threadIdx.x == 0)
    alpha[0] = c * c / (cm(cmax, 2) * kQ);
  if (i >= numel) return;
  float x[N];
  int m[N];
  ldv(in, i, x);
#pragma unroll
  for (int k = 0; k < N; ++k) x[k] = fake_quantize_b(x[k], c, m[k], bit, symmetry != 0);
  stv(out, i, x);
  or_mask<N>(cmask, i, m);
}

template <typename T>
__global__ void __launch_bounds__(256)
dequantize_b_kernel(T* __restrict__ f, const int8_t* __restrict__ q, const T* __restrict__ cmax,
                    long numel) {
  constexpr int N = Vec<T>::N;
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * N;
  if (i >= numel) return;
  const float c = cm(cmax);
  int qv[N];
  float x[N];
  ldq<N>(q, i, qv);
#pragma unroll
  for (int k = 0; k < N; ++k) x[k] = dequantize_b(qv[k], c);
  stv(f, i, x);
}

// ---------------------------------------------------------------------------------
// layer norm (normalize_kernels.cu:40-380): var = E[x^2] - E[x]^2 + 1e-8.
// One wavefront per row, 4 rows per workgroup; the row is read twice (the second read
// is served by the cache).
// ---------------------------------------------------------------------------------
template <typename T, bool I8>
__global__ void __launch_bounds__(256)
layer_norm_b_kernel(T* ln_res, int8_t* __restrict__ q_out, uint8_t* cmask, T* __restrict__ vars,
                    T* __restrict__ means, const T* inp, const T* __restrict__ gamma,
                    const T* __restrict__ beta, const T* __restrict__ cmax_out, int rows,
                    int hidden) {
  constexpr int N = Vec<T>::N;
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const long base = (long)row * hidden;
  float s = 0.f, s2 = 0.f;
  for (int e = lane * N; e < hidden; e += 64 * N) {
    float x[N];
    ldv(inp, base + e, x);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      s += x[k];
      s2 += x[k] * x[k];
    }
  }
  const float mean = wave_sum(s) / (float)hidden;
  const float var = wave_sum(s2) / (float)hidden - mean * mean + kLnEps;
  const float rstd = rsqrtf(var);
  const float c = I8 ? cm(cmax_out) : 0.f;
  for (int e = lane * N; e < hidden; e += 64 * N) {
    float x[N], g[N], b[N];
    ldv(inp, base + e, x);
    ldv(gamma, e, g);
    ldv(beta, e, b);
#pragma unroll
    for (int k = 0; k < N; ++k) x[k] = (x[k] - mean) * rstd * g[k] + b[k];
    if (I8) {
      int qv[N], m[N];
#pragma unroll
      for (int k = 0; k < N; ++k) qv[k] = quantize_b(x[k], c, m[k], 2);
      stq<N>(q_out, base + e, qv);
      or_mask<N>(cmask, base + e, m);
    } else {
      stv(ln_res, base + e, x);
    }
  }
  if (lane == 0) {
    if (vars != nullptr) TT<T>::st(vars, row, var);
    if (means != nullptr) TT<T>::st(means, row, mean);
  }
}

// ---------------------------------------------------------------------------------
// masked softmax (softmax_kernels.cu:35-279): one wavefront per (batch, head, query) row,
// to_len <= 1024 -> at most 16 values per lane in registers.
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
attn_softmax_b_kernel(T* vals, const T* __restrict__ mask, long rows, int heads, int from_len,
                      int to_len, int mask_future) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int qi = (int)(row % from_len);
  const long b = row / ((long)from_len * heads);
  T* p = vals + row * to_len;
  float x[16];
  float mx = kFloatInfNeg;
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int j = it * 64 + lane;
    float v = kFloatInfNeg;
    if (j < to_len) {
      if (!(mask_future && j > qi)) {
        v = TT<T>::ld(p, j);
        if (mask != nullptr) v += TT<T>::ld(mask, b * to_len + j);
      }
    }
    x[it] = v;
    mx = fmaxf(mx, v);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int j = it * 64 + lane;
    x[it] = j < to_len ? __expf(x[it] - mx) : 0.f;
    sum += x[it];
  }
  const float inv = 1.0f / (wave_sum(sum) + kSoftmaxEps);
#pragma unroll
  for (int it = 0; it < 16; ++it) {
    const int j = it * 64 + lane;
    if (j < to_len) TT<T>::st(p, j, x[it] * inv);
  }
}

// ---------------------------------------------------------------------------------
// head split / merge (transform_kernels.cu)
// ---------------------------------------------------------------------------------
// int8 [d0, d1, d2, d3, d4] -> T [d2, d0, d3, d1, d4], dequantise + bias (+ fake quant)
template <typename T>
__global__ void __launch_bounds__(256)
quant_bias_add_transform_20314_kernel(T* __restrict__ out, const int8_t* __restrict__ in,
                                      const T* __restrict__ bias, const T* __restrict__ cmax,
                                      const T* __restrict__ out_cmax, int d0, int d1, int d2,
                                      int d3, int d4, long nvec) {
  constexpr int N = Vec<T>::N;
  const long v = (long)blockIdx.x * 256 + threadIdx.x;
  if (v >= nvec) return;
  const long i = v * N;
  const int d34 = d3 * d4;
  const int e34 = (int)(i % d34);
  long r = i / d34;
  const int i2 = (int)(r % d2);
  r /= d2;
  const int i1 = (int)(r % d1);
  const int i0 = (int)(r / d1);
  const int i3 = e34 / d4, i4 = e34 % d4;
  const float c = cm(cmax);
  int qv[N];
  float b[N], x[N];
  ldq<N>(in, i, qv);
  ldv(bias, (long)i2 * d34 + e34, b);
#pragma unroll
  for (int k = 0; k < N; ++k) x[k] = deq_bias<T>(qv[k], c, b[k]);
  if (out_cmax != nullptr) {
    const float oc = cm(out_cmax);
    int m;
#pragma unroll
    for (int k = 0; k < N; ++k) x[k] = fake_quantize_b(x[k], oc, m, 6, true);
  }
  const long o = ((((long)i2 * d0 + i0) * d3 + i3) * d1 + i1) * d4 + i4;
  stv(out, o, x);
}

// T [d0, d1, d2, d3, d4] -> T [d2, d0, d3, d1, d4] with bias [d2, d3, d4] added
// (launch_bias_add_transform_20314, transform_kernels.cu:140-235); T=half adds in half.
template <typename T>
__global__ void __launch_bounds__(256)
bias_add_transform_20314_kernel(T* __restrict__ out, const T* __restrict__ in,
                                const T* __restrict__ bias, int d0, int d1, int d2, int d3,
                                int d4, long nvec) {
  constexpr int N = Vec<T>::N;
  const long v = (long)blockIdx.x * 256 + threadIdx.x;
  if (v >= nvec) return;
  const long i = v * N;
  const int d34 = d3 * d4;
  const int e34 = (int)(i % d34);
  long r = i / d34;
  const int i2 = (int)(r % d2);
  r /= d2;
  const int i1 = (int)(r % d1);
  const int i0 = (int)(r / d1);
  const int i3 = e34 / d4, i4 = e34 % d4;
  float x[N], b[N];
  ldv(in, i, x);
  ldv(bias, (long)i2 * d34 + e34, b);
#pragma unroll
  for (int k = 0; k < N; ++k) x[k] = TT<T>::rnd(x[k] + b[k]);
  const long o = ((((long)i2 * d0 + i0) * d3 + i3) * d1 + i1) * d4 + i4;
  stv(out, o, x);
}

// [sz0, sz1_1, sz2] ++ [sz0, sz1_2, sz2] -> [sz0, sz1_1 + sz1_2, sz2] along dim 1
// (launch_concat3_dim1, general_kernels.cu:187-234)
template <typename T>
__global__ void __launch_bounds__(256)
concat3_dim1_kernel(const T* __restrict__ inp1, const T* __restrict__ inp2, T* __restrict__ out,
                    int sz2, int sz1_1, int sz1_2, long nvec) {
  constexpr int N = Vec<T>::N;
  const long v = (long)blockIdx.x * 256 + threadIdx.x;
  if (v >= nvec) return;
  const long i = v * N;
  const int i2 = (int)(i % sz2);
  long r = i / sz2;
  const int i1 = (int)(r % (sz1_1 + sz1_2));
  const long i0 = r / (sz1_1 + sz1_2);
  float x[N];
  if (i1 < sz1_1)
    ldv(inp1, (i0 * sz1_1 + i1) * sz2 + i2, x);
  else
    ldv(inp2, (i0 * sz1_2 + (i1 - sz1_1)) * sz2 + i2, x);
  stv(out, i, x);
}

// T [tc, b, nh, s, ad] -> [b, s, tc, nh, ad], optionally quantised
template <typename T, bool QUANT>
__global__ void __launch_bounds__(256)
transform4d_0213_kernel(T* __restrict__ out, int8_t* __restrict__ out_q, uint8_t* cmask,
                        const T* __restrict__ in, const T* __restrict__ cmax, int batch, int seq,
                        int tc, int nhead, int hd, long nvec) {
  constexpr int N = Vec<T>::N;
  const long v = (long)blockIdx.x * 256 + threadIdx.x;
  if (v >= nvec) return;
  const long i = v * N;
  const int id = (int)(i % hd);
  long r = i / hd;
  const int is = (int)(r % seq);
  r /= seq;
  const int ih = (int)(r % nhead);
  r /= nhead;
  const int ib = (int)(r % batch);
  const int it = (int)(r / batch);
  const long o = ((((long)ib * seq + is) * tc + it) * nhead + ih) * hd + id;
  float x[N];
  ldv(in, i, x);
  if (QUANT) {
    const float c = cm(cmax);
    int qv[N], m[N];
#pragma unroll
    for (int k = 0; k < N; ++k) qv[k] = quantize_b(x[k], c, m[k], 2);
    stq<N>(out_q, o, qv);
    or_mask<N>(cmask, o, m);
  } else {
    stv(out, o, x);
  }
}

// ---------------------------------------------------------------------------------
// bias / activation / residual epilogues (dropout_kernels.cu) with dropout ratio 0
// ---------------------------------------------------------------------------------
template <int N>
__device__ __forceinline__ void set_dropout_mask(uint8_t* p, long i, bool assign) {
  if (p == nullptr) return;
  int one[N];
#pragma unroll
  for (int k = 0; k < N; ++k) one[k] = 1;
  if (assign) {
    if (N == 8)
      *reinterpret_cast<uint2*>(p + i) = make_uint2(0x01010101u, 0x01010101u);
    else
      *reinterpret_cast<uint32_t*>(p + i) = 0x01010101u;
  } else {
    or_mask<N>(p, i, one);
  }
}

// MODE 0: out = in (launch_ls_dropout); 1: (in + bias) + residual; 2: act(in + bias)
template <typename T, int MODE, int ACT>
__global__ void __launch_bounds__(256)
dropout_b_kernel(T* out, const T* in, uint8_t* mask, const T* __restrict__ bias,
                 const T* residual, long numel, int dim) {
  constexpr int N = Vec<T>::N;
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * N;
  if (i >= numel) return;
  float x[N];
  ldv(in, i, x);
  if (MODE != 0) {
    float b[N];
    ldv(bias, i % dim, b);
#pragma unroll
    for (int k = 0; k < N; ++k) x[k] = TT<T>::rnd(x[k] + b[k]);
    if (MODE == 1) {
      float r[N];
      ldv(residual, i, r);
#pragma unroll
      for (int k = 0; k < N; ++k) x[k] += r[k];
    } else {
#pragma unroll
      for (int k = 0; k < N; ++k) x[k] = act_b<T, ACT>(x[k]);
    }
  }
  stv(out, i, x);
  set_dropout_mask<N>(mask, i, true);
}

// OUT 0: int8 codes (launch_ls_quant_dropout_act_bias); 1: fake-quantised T
// (launch_ls_fakequant_dropout_act_bias).  `cmax_out` dequantises the input codes,
// `cmax_in` (the next GEMM's input clip) quantises the result, as in the reference.
template <typename T, int ACT, int OUT>
__global__ void __launch_bounds__(256)
quant_act_bias_b_kernel(int8_t* __restrict__ qout, T* __restrict__ fout, uint8_t* cmask_in,
                        uint8_t* dropout_mask, const int8_t* __restrict__ qin,
                        const T* __restrict__ bias, const T* __restrict__ cmax_out,
                        const T* __restrict__ cmax_in, long numel, int dim, int symmetry) {
  constexpr int N = Vec<T>::N;
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * N;
  if (i >= numel) return;
  const float co = cm(cmax_out), ci = cm(cmax_in);
  int qv[N], m[N];
  float b[N], x[N];
  ldq<N>(qin, i, qv);
  ldv(bias, i % dim, b);
#pragma unroll
  for (int k = 0; k < N; ++k) x[k] = act_b<T, ACT>(deq_bias<T>(qv[k], co, b[k]));
  if (OUT == 0) {
#pragma unroll
    for (int k = 0; k < N; ++k) qv[k] = quantize_b(x[k], ci, m[k], 2);
    stq<N>(qout, i, qv);
  } else {
#pragma unroll
    for (int k = 0; k < N; ++k) x[k] = fake_quantize_b(x[k], ci, m[k], 2, symmetry != 0);
    stv(fout, i, x);
  }
  or_mask<N>(cmask_in, i, m);
  set_dropout_mask<N>(dropout_mask, i, false);
}

template <typename T>
__global__ void __launch_bounds__(256)
quant_res_bias_b_kernel(T* out, uint8_t* mask, const int8_t* __restrict__ qin,
                        const T* __restrict__ cmax, const T* __restrict__ bias,
                        const T* residual, long numel, int dim) {
  constexpr int N = Vec<T>::N;
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * N;
  if (i >= numel) return;
  const float c = cm(cmax);
  int qv[N];
  float b[N], r[N], x[N];
  ldq<N>(qin, i, qv);
  ldv(bias, i % dim, b);
  ldv(residual, i, r);
#pragma unroll
  for (int k = 0; k < N; ++k) x[k] = deq_bias<T>(qv[k], c, b[k]) + r[k];
  stv(out, i, x);
  set_dropout_mask<N>(mask, i, false);
}

template <typename T>
int check_vec(long numel, const char* what) {
  constexpr int N = Vec<T>::N;
  if (numel <= 0 || numel % N != 0) {
    static thread_local std::string msg;
    msg = std::string(what) + (N == 8 ? ": violate numel % 8 = 0" : ": violate numel % 4 = 0");
    return lsh_fail(LSH_ERR_INVALID, msg.c_str());
  }
  return LSH_OK;
}

int check_ratio(float ratio, const char* what) {
  if (ratio != 0.f) {
    static thread_local std::string msg;
    msg = std::string(what) + ": dropout ratio must be 0 (forward-only inference build)";
    return lsh_fail(LSH_ERR_UNSUPPORTED, msg.c_str());
  }
  return LSH_OK;
}

}  // namespace

// ---------------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------------
template <typename T>
int opb_quantize(int8_t* q, uint8_t* cmask, float* alpha, const T* f, const T* cmax, long numel,
                 int alpha_count, int bit, hipStream_t s) {
  if (!q || !f || !cmax) return lsh_fail(LSH_ERR_INVALID, "launch_quantize: null pointer");
  if (int rc = check_vec<T>(numel, "launch_quantize")) return rc;
  quantize_b_kernel<T><<<grid_for(numel / Vec<T>::N), 256, 0, s>>>(q, cmask, alpha, f, cmax,
                                                                   numel, alpha_count, bit);
  return lsh_check_launch("quantize_b_kernel");
}

template <typename T>
int opb_fake_quantize(uint8_t* cmask, float* alpha, T* out, const T* in, const T* cmax,
                      long numel, int bit, bool symmetry, hipStream_t s) {
  if (!out || !in || !cmax) return lsh_fail(LSH_ERR_INVALID, "launch_fake_quantize: null pointer");
  if (int rc = check_vec<T>(numel, "launch_fake_quantize")) return rc;
  fake_quantize_b_kernel<T><<<grid_for(numel / Vec<T>::N), 256, 0, s>>>(
      cmask, alpha, out, in, cmax, numel, bit, symmetry ? 1 : 0);
  return lsh_check_launch("fake_quantize_b_kernel");
}

template <typename T>
int opb_dequantize(T* f, const int8_t* q, const T* cmax, long numel, hipStream_t s) {
  if (!f || !q || !cmax) return lsh_fail(LSH_ERR_INVALID, "launch_dequantize: null pointer");
  if (int rc = check_vec<T>(numel, "launch_dequantize")) return rc;
  dequantize_b_kernel<T><<<grid_for(numel / Vec<T>::N), 256, 0, s>>>(f, q, cmax, numel);
  return lsh_check_launch("dequantize_b_kernel");
}

template <typename T>
int opb_layer_norm(T* ln_res, int8_t* q_out, uint8_t* cmask, T* vars, T* means, const T* inp,
                   const T* gamma, const T* beta, const T* cmax_out, int rows, int hidden,
                   hipStream_t s) {
  const bool i8 = q_out != nullptr;
  if (!inp || !gamma || !beta || (!i8 && !ln_res) || (i8 && !cmax_out))
    return lsh_fail(LSH_ERR_INVALID, "launch_layer_norm: null pointer");
  if (rows <= 0 || hidden <= 0 || hidden % Vec<T>::N != 0)
    return lsh_fail(LSH_ERR_INVALID, sizeof(T) == 2 ? "violate hidden_dim % 8 = 0"
                                                    : "violate hidden_dim % 4 = 0");
  const int grid = (rows + 3) / 4;
  if (i8)
    layer_norm_b_kernel<T, true><<<grid, 256, 0, s>>>(nullptr, q_out, cmask, vars, means, inp,
                                                      gamma, beta, cmax_out, rows, hidden);
  else
    layer_norm_b_kernel<T, false><<<grid, 256, 0, s>>>(ln_res, nullptr, nullptr, vars, means, inp,
                                                       gamma, beta, nullptr, rows, hidden);
  return lsh_check_launch("layer_norm_b_kernel");
}

template <typename T>
int opb_attn_softmax(T* vals, const T* mask, int batch, int heads, int from_len, int to_len,
                     bool mask_future, hipStream_t s) {
  if (!vals || batch <= 0 || heads <= 0 || from_len <= 0 || to_len <= 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_attn_softmax: bad arguments");
  if (to_len > 1024)
    return lsh_fail(LSH_ERR_UNSUPPORTED,
                    "Sequence length greater than 512 is currently not supported");
  const long rows = (long)batch * heads * from_len;
  attn_softmax_b_kernel<T><<<(int)((rows + 3) / 4), 256, 0, s>>>(vals, mask, rows, heads, from_len,
                                                                 to_len, mask_future ? 1 : 0);
  return lsh_check_launch("attn_softmax_b_kernel");
}

template <typename T>
int opb_quant_bias_add_transform_20314(T* out, uint8_t* cmask, const int8_t* in, const T* bias,
                                       const T* cmax, int d0, int d1, int d2, int d3, int d4,
                                       hipStream_t s, const T* out_cmax) {
  (void)cmask;  // the reference computes these bits into a local it never stores
  if (!out || !in || !bias || !cmax)
    return lsh_fail(LSH_ERR_INVALID, "launch_quant_bias_add_transform_20314: null pointer");
  if (d0 <= 0 || d1 <= 0 || d2 <= 0 || d3 <= 0 || d4 <= 0 || d4 % Vec<T>::N != 0)
    return lsh_fail(LSH_ERR_INVALID,
                    "launch_quant_bias_add_transform_20314: dim_4 must be a multiple of the "
                    "vector width");
  const long nvec = (long)d0 * d1 * d2 * d3 * d4 / Vec<T>::N;
  quant_bias_add_transform_20314_kernel<T><<<grid_for(nvec), 256, 0, s>>>(
      out, in, bias, cmax, out_cmax, d0, d1, d2, d3, d4, nvec);
  return lsh_check_launch("quant_bias_add_transform_20314_kernel");
}

template <typename T>
int opb_bias_add_transform_20314(T* out, const T* in, const T* bias, int d0, int d1, int d2,
                                 int d3, int d4, hipStream_t s) {
  if (!out || !in || !bias)
    return lsh_fail(LSH_ERR_INVALID, "launch_bias_add_transform_20314: null pointer");
  if (d0 <= 0 || d1 <= 0 || d2 <= 0 || d3 <= 0 || d4 <= 0 || d4 % Vec<T>::N != 0)
    return lsh_fail(LSH_ERR_INVALID,
                    "launch_bias_add_transform_20314: dim_4 must be a multiple of the vector "
                    "width");
  const long nvec = (long)d0 * d1 * d2 * d3 * d4 / Vec<T>::N;
  bias_add_transform_20314_kernel<T><<<grid_for(nvec), 256, 0, s>>>(out, in, bias, d0, d1, d2,
                                                                    d3, d4, nvec);
  return lsh_check_launch("bias_add_transform_20314_kernel");
}

template <typename T>
int opb_concat3_dim1(const T* inp1, const T* inp2, T* out, int sz0, int sz2, int sz1_1,
                     int sz1_2, hipStream_t s) {
  if (!out || (!inp1 && sz1_1 > 0) || (!inp2 && sz1_2 > 0))
    return lsh_fail(LSH_ERR_INVALID, "launch_concat3_dim1: null pointer");
  if (sz0 <= 0 || sz2 <= 0 || sz1_1 < 0 || sz1_2 < 0 || sz1_1 + sz1_2 == 0 ||
      sz2 % Vec<T>::N != 0)
    return lsh_fail(LSH_ERR_INVALID,
                    "launch_concat3_dim1: the last dimension must be a multiple of the vector "
                    "width");
  const long nvec = (long)sz0 * (sz1_1 + sz1_2) * sz2 / Vec<T>::N;
  concat3_dim1_kernel<T><<<grid_for(nvec), 256, 0, s>>>(inp1, inp2, out, sz2, sz1_1, sz1_2, nvec);
  return lsh_check_launch("concat3_dim1_kernel");
}

template <typename T>
int opb_transform4d_0213(T* out, int8_t* out_q, uint8_t* cmask, const T* vals, const T* cmax,
                         int batch, int seq, int hidden, int nhead, int tc, hipStream_t s) {
  const bool quant = out_q != nullptr;
  if (!vals || (!quant && !out) || (quant && !cmax))
    return lsh_fail(LSH_ERR_INVALID, "launch_transform4d_0213: null pointer");
  if (batch <= 0 || seq <= 0 || hidden <= 0 || nhead <= 0 || tc <= 0 || hidden % nhead != 0 ||
      (hidden / nhead) % Vec<T>::N != 0)
    return lsh_fail(LSH_ERR_INVALID,
                    "launch_transform4d_0213: head dim must be a multiple of the vector width");
  const int hd = hidden / nhead;
  const long nvec = (long)batch * seq * tc * hidden / Vec<T>::N;
  if (quant)
    transform4d_0213_kernel<T, true><<<grid_for(nvec), 256, 0, s>>>(
        nullptr, out_q, cmask, vals, cmax, batch, seq, tc, nhead, hd, nvec);
  else
    transform4d_0213_kernel<T, false><<<grid_for(nvec), 256, 0, s>>>(
        out, nullptr, nullptr, vals, nullptr, batch, seq, tc, nhead, hd, nvec);
  return lsh_check_launch("transform4d_0213_kernel");
}

template <typename T>
int opb_dropout(T* out, const T* vals, uint8_t* mask, long total, float ratio, hipStream_t s) {
  if (!out || !vals) return lsh_fail(LSH_ERR_INVALID, "launch_ls_dropout: null pointer");
  if (int rc = check_ratio(ratio, "launch_ls_dropout")) return rc;
  if (int rc = check_vec<T>(total, "launch_ls_dropout")) return rc;
  dropout_b_kernel<T, 0, 0><<<grid_for(total / Vec<T>::N), 256, 0, s>>>(out, vals, mask, nullptr,
                                                                        nullptr, total, 1);
  return lsh_check_launch("dropout_b_kernel");
}

template <typename T>
int opb_dropout_res_bias(T* out, const T* vals, uint8_t* mask, const T* bias, const T* residual,
                         long total, int dim, float ratio, hipStream_t s) {
  if (!out || !vals || !bias || !residual)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_dropout_res_bias: null pointer");
  if (int rc = check_ratio(ratio, "launch_ls_dropout_res_bias")) return rc;
  if (int rc = check_vec<T>(total, "launch_ls_dropout_res_bias")) return rc;
  if (dim <= 0 || dim % Vec<T>::N != 0 || total % dim != 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_dropout_res_bias: bad dim");
  dropout_b_kernel<T, 1, 0><<<grid_for(total / Vec<T>::N), 256, 0, s>>>(out, vals, mask, bias,
                                                                        residual, total, dim);
  return lsh_check_launch("dropout_b_kernel");
}

template <typename T>
int opb_dropout_act_bias(int act, T* out, const T* vals, uint8_t* mask, const T* bias, long total,
                         int dim, float ratio, hipStream_t s) {
  if (!out || !vals || !bias)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_dropout_act_bias: null pointer");
  if (int rc = check_ratio(ratio, "launch_ls_dropout_act_bias")) return rc;
  if (int rc = check_vec<T>(total, "launch_ls_dropout_act_bias")) return rc;
  if (dim <= 0 || dim % Vec<T>::N != 0 || total % dim != 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_dropout_act_bias: bad dim");
  const int grid = grid_for(total / Vec<T>::N);
  if (act == 0)
    dropout_b_kernel<T, 2, 0><<<grid, 256, 0, s>>>(out, vals, mask, bias, nullptr, total, dim);
  else
    dropout_b_kernel<T, 2, 1><<<grid, 256, 0, s>>>(out, vals, mask, bias, nullptr, total, dim);
  return lsh_check_launch("dropout_b_kernel");
}

template <typename T>
int opb_quant_dropout_act_bias(int act, int8_t* qout, T* fout, uint8_t* cmask_out,
                               uint8_t* cmask_in, uint8_t* dropout_mask, const int8_t* qin,
                               const T* bias, const T* cmax_out, const T* cmax_in, long total,
                               int dim, float ratio, bool symmetry, hipStream_t s) {
  (void)cmask_out;  // unused by the reference kernels too
  if ((!qout && !fout) || !qin || !bias || !cmax_out || !cmax_in)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_quant_dropout_act_bias: null pointer");
  if (int rc = check_ratio(ratio, "launch_ls_quant_dropout_act_bias")) return rc;
  if (int rc = check_vec<T>(total, "launch_ls_quant_dropout_act_bias")) return rc;
  if (dim <= 0 || dim % Vec<T>::N != 0 || total % dim != 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_quant_dropout_act_bias: bad dim");
  const int grid = grid_for(total / Vec<T>::N);
  const int sym = symmetry ? 1 : 0;
#define LSH_QAB(ACT, OUT)                                                                      \
  quant_act_bias_b_kernel<T, ACT, OUT><<<grid, 256, 0, s>>>(                                    \
      qout, fout, cmask_in, dropout_mask, qin, bias, cmax_out, cmax_in, total, dim, sym)
  if (qout != nullptr) {
    if (act == 0) LSH_QAB(0, 0); else LSH_QAB(1, 0);
  } else {
    if (act == 0) LSH_QAB(0, 1); else LSH_QAB(1, 1);
  }
#undef LSH_QAB
  return lsh_check_launch("quant_act_bias_b_kernel");
}

template <typename T>
int opb_quant_dropout_res_bias(T* out, uint8_t* mask, const int8_t* qvals, const T* cmax,
                               const T* bias, const T* residual, long total, int dim, float ratio,
                               hipStream_t s) {
  if (!out || !qvals || !cmax || !bias || !residual)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_quant_dropout_res_bias: null pointer");
  if (int rc = check_ratio(ratio, "launch_ls_quant_dropout_res_bias")) return rc;
  if (int rc = check_vec<T>(total, "launch_ls_quant_dropout_res_bias")) return rc;
  if (dim <= 0 || dim % Vec<T>::N != 0 || total % dim != 0)
    return lsh_fail(LSH_ERR_INVALID, "launch_ls_quant_dropout_res_bias: bad dim");
  quant_res_bias_b_kernel<T><<<grid_for(total / Vec<T>::N), 256, 0, s>>>(out, mask, qvals, cmax,
                                                                         bias, residual, total,
                                                                         dim);
  return lsh_check_launch("quant_res_bias_b_kernel");
}

#define LSH_INST(T)                                                                              \
  template int opb_quantize<T>(int8_t*, uint8_t*, float*, const T*, const T*, long, int, int,    \
                               hipStream_t);                                                     \
  template int opb_fake_quantize<T>(uint8_t*, float*, T*, const T*, const T*, long, int, bool,   \
                                    hipStream_t);                                                \
  template int opb_dequantize<T>(T*, const int8_t*, const T*, long, hipStream_t);                \
  template int opb_layer_norm<T>(T*, int8_t*, uint8_t*, T*, T*, const T*, const T*, const T*,    \
                                 const T*, int, int, hipStream_t);                               \
  template int opb_attn_softmax<T>(T*, const T*, int, int, int, int, bool, hipStream_t);         \
  template int opb_quant_bias_add_transform_20314<T>(T*, uint8_t*, const int8_t*, const T*,      \
                                                     const T*, int, int, int, int, int,          \
                                                     hipStream_t, const T*);                     \
  template int opb_transform4d_0213<T>(T*, int8_t*, uint8_t*, const T*, const T*, int, int, int, \
                                       int, int, hipStream_t);                                   \
  template int opb_bias_add_transform_20314<T>(T*, const T*, const T*, int, int, int, int, int,  \
                                               hipStream_t);                                     \
  template int opb_concat3_dim1<T>(const T*, const T*, T*, int, int, int, int, hipStream_t);     \
  template int opb_dropout<T>(T*, const T*, uint8_t*, long, float, hipStream_t);                 \
  template int opb_dropout_res_bias<T>(T*, const T*, uint8_t*, const T*, const T*, long, int,    \
                                       float, hipStream_t);                                      \
  template int opb_dropout_act_bias<T>(int, T*, const T*, uint8_t*, const T*, long, int, float,  \
                                       hipStream_t);                                             \
  template int opb_quant_dropout_act_bias<T>(int, int8_t*, T*, uint8_t*, uint8_t*, uint8_t*,     \
                                             const int8_t*, const T*, const T*, const T*, long,  \
                                             int, float, bool, hipStream_t);                     \
  template int opb_quant_dropout_res_bias<T>(T*, uint8_t*, const int8_t*, const T*, const T*,    \
                                             const T*, long, int, float, hipStream_t);
LSH_INST(float)
LSH_INST(__half)
#undef LSH_INST

}  // namespace lsh
