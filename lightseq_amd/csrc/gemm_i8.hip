// int8 x int8 -> int32 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8),
// with optional requantising epilogue.
//
//   C[M,N] = epilogue( sum_k A[M,k] * W[N,k] )        A, W: K-contiguous int8
//
// Replaces the cuBLASLt int8 GEMMs and their tuned-algorithm table
// (inference/model/cublas_helper.cc:31-225,361-489, cublas_algo_map.cc).
//
// Tiling.  A workgroup of 256 threads (4 wavefronts, 2x2) owns a BM x BN tile of C
// and walks K in steps of 128 bytes.  Both operand tiles are staged in LDS,
// double buffered, as rows of 128 bytes whose eight 16-byte chunks are XOR
// swizzled so that the 16-byte per-lane MFMA operand reads are bank-conflict free.
// The W tile is the MFMA "A" operand and the activation tile the "B" operand, so
// that consecutive accumulator registers of a lane run along N; the W rows fed to
// the MFMA are permuted so that the 16 accumulators of a lane are 16 *adjacent*
// columns of C (one 16-byte store for int8 output).
#include "ls_device.cuh"
#include "ls_launch.h"

#include <string>

namespace lsh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 128;  // bytes of K per LDS stage

// swizzle keys (3 bits) of a tile row
__device__ __forceinline__ int key_act(int row) { return row & 7; }
__device__ __forceinline__ int key_wgt(int row) { return (row & 3) | (((row >> 4) & 1) << 2); }
// MFMA row r (0..31) of the weight operand -> local column of C, chosen so that the
// accumulators c[0..15] of lane (l%32, g=l/32) are columns 16g .. 16g+15.
__device__ __forceinline__ int sigma(int r) { return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3); }

struct EpiI32 {
  int32_t* C;
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    int32_t* p = C + m * N + n;
    if (full) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<int4*>(p + 4 * q) =
            make_int4(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]);
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (n + i < N) p[i] = c[i];
    }
  }
  __host__ __device__ static bool vec_ok(int N, const void* C) {
    return N % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0;
  }
};

struct EpiI8 {
  int8_t* C;
  float alpha;
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    int8_t* p = C + m * N + n;
    if (full) {
      uint4 o;
      o.x = pack4_i8(requant_acc(c[0], alpha), requant_acc(c[1], alpha), requant_acc(c[2], alpha),
                     requant_acc(c[3], alpha));
      o.y = pack4_i8(requant_acc(c[4], alpha), requant_acc(c[5], alpha), requant_acc(c[6], alpha),
                     requant_acc(c[7], alpha));
      o.z = pack4_i8(requant_acc(c[8], alpha), requant_acc(c[9], alpha),
                     requant_acc(c[10], alpha), requant_acc(c[11], alpha));
      o.w = pack4_i8(requant_acc(c[12], alpha), requant_acc(c[13], alpha),
                     requant_acc(c[14], alpha), requant_acc(c[15], alpha));
      *reinterpret_cast<uint4*>(p) = o;
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (n + i < N) p[i] = (int8_t)requant_acc(c[i], alpha);
    }
  }
  __host__ __device__ static bool vec_ok(int N, const void* C) {
    return N % 16 == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0;
  }
};

// Load one BK-wide stage of a ROWS-row tile (row stride K bytes in HBM) into
// registers: ROWS*8 chunks of 16 B spread over 256 threads.
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

template <int BM, int BN, typename Epi>
__global__ void __launch_bounds__(256)
gemm_i8_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, Epi epi, int M, int N,
               int K, int tiles_m, int tiles_n, bool vec_store) {
  constexpr int TM = BM / 2, TN = BN / 2;      // wavefront tile
  constexpr int MB = TM / 32, NB = TN / 32;    // MFMA blocks per wavefront tile
  extern __shared__ __align__(16) int8_t smem[];
  constexpr int kStage = (BM + BN) * kBK;  // bytes per LDS stage: A tile then W tile

  // Workgroups are dealt round-robin to the 8 XCDs; renumber them so that each XCD
  // (own L2) works on a contiguous run of tiles, and walk tiles in column-major
  // order of 8-tile-tall groups so a run shares W columns and A rows.
  const int nblk = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int per = nblk / 8, rem = nblk % 8;
    const int xcd = pid % 8, loc = pid / 8;
    pid = xcd * per + (xcd < rem ? xcd : rem) + loc;
  }
  constexpr int GROUP = 8;
  const int group_sz = GROUP * tiles_n;
  const int gid = pid / group_sz;
  const int first_m = gid * GROUP;
  const int gm = min(tiles_m - first_m, GROUP);
  const int tile_m = first_m + (pid % group_sz) % gm;
  const int tile_n = (pid % group_sz) / gm;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  v16i acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) acc[i][j] = (v16i)0;

  v4i ra[BM / 32], rw[BN / 32];
  const int nk = (K + kBK - 1) / kBK;
  load_tile<BM>(A, m0, M, K, 0, tid, ra);
  load_tile<BN>(W, n0, N, K, 0, tid, rw);
  store_tile<BM, false>(smem, tid, ra);
  store_tile<BN, true>(smem + BM * kBK, tid, rw);
  __syncthreads();

  // per-lane LDS row offsets of the MFMA operands
  int a_off[MB], w_off[NB], a_key[MB], w_key[NB];
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int row = wm * TM + i * 32 + l32;
    a_off[i] = row * kBK;
    a_key[i] = key_act(row);
  }
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int row = wn * TN + j * 32 + sigma(l32);
    w_off[j] = row * kBK;
    w_key[j] = key_wgt(row);
  }

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      load_tile<BM>(A, m0, M, K, (kt + 1) * kBK, tid, ra);
      load_tile<BN>(W, n0, N, K, (kt + 1) * kBK, tid, rw);
    }
    const int8_t* pa = smem + cur * kStage;
    const int8_t* pw = pa + BM * kBK;
#pragma unroll
    for (int ks = 0; ks < kBK / 32; ++ks) {
      const int chunk = 2 * ks + g;
      v4i bv[MB], av[NB];
#pragma unroll
      for (int i = 0; i < MB; ++i)
        bv[i] = *reinterpret_cast<const v4i*>(pa + a_off[i] + ((chunk ^ a_key[i]) << 4));
#pragma unroll
      for (int j = 0; j < NB; ++j)
        av[j] = *reinterpret_cast<const v4i*>(pw + w_off[j] + ((chunk ^ w_key[j]) << 4));
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[j], bv[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) {
      int8_t* nxt = smem + (cur ^ 1) * kStage;
      store_tile<BM, false>(nxt, tid, ra);
      store_tile<BN, true>(nxt + BM * kBK, tid, rw);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const long m = m0 + wm * TM + i * 32 + l32;
    if (m < M) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int n = n0 + wn * TN + j * 32 + 16 * g;
        if (n < N) epi.store16(m, n, N, acc[i][j], vec_store && n + 16 <= N);
      }
    }
  }
}

template <int BM, int BN, typename Epi>
static int launch_tile(const int8_t* A, const int8_t* W, Epi epi, int M, int N, int K,
                       bool vec_store, hipStream_t s) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const size_t smem = 2 * (size_t)(BM + BN) * kBK;
  auto kern = gemm_i8_kernel<BM, BN, Epi>;
  static bool attr_set = false;  // per instantiation
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return lsh_check_hip(e, "hipFuncSetAttribute(gemm_i8_kernel)");
    attr_set = true;
  }
  kern<<<tiles_m * tiles_n, 256, smem, s>>>(A, W, epi, M, N, K, tiles_m, tiles_n, vec_store);
  return lsh_check_launch("gemm_i8_kernel");
}

// Picks the tile that wastes the fewest matrix-core cycles on 256 compute units:
// cost = (#rounds of 256 workgroups) x (work per tile), penalising small tiles for
// their higher LDS traffic per MAC.  Returns an index into kTiles.
struct TileCand { int bm, bn; double eff; };
static const TileCand kTiles[3] = {{256, 256, 1.0}, {256, 128, 0.92}, {128, 128, 0.80}};

static int select_tile(int M, int N) {
  int best = 2;
  double best_cost = 1e300;
  for (int c = 0; c < 3; ++c) {
    const long tiles =
        (long)((M + kTiles[c].bm - 1) / kTiles[c].bm) * ((N + kTiles[c].bn - 1) / kTiles[c].bn);
    const long rounds = (tiles + 255) / 256;
    const double cost = (double)rounds * kTiles[c].bm * kTiles[c].bn / kTiles[c].eff;
    if (cost < best_cost) { best_cost = cost; best = c; }
  }
  return best;
}

template <typename Epi>
static int dispatch(const int8_t* A, const int8_t* W, Epi epi, int M, int N, int K,
                    const void* Cptr, hipStream_t s) {
  if (M <= 0 || N <= 0 || K <= 0 || !A || !W || !Cptr)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm: bad arguments");
  if (K % 16 != 0) return lsh_fail(LSH_ERR_UNSUPPORTED, "int8 gemm: K must be a multiple of 16");
  if (((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W)) & 15u) != 0)
    return lsh_fail(LSH_ERR_INVALID, "int8 gemm: operands must be 16-byte aligned");
  const bool vec_store = Epi::vec_ok(N, Cptr);
  switch (select_tile(M, N)) {
    case 0: return launch_tile<256, 256, Epi>(A, W, epi, M, N, K, vec_store, s);
    case 1: return launch_tile<256, 128, Epi>(A, W, epi, M, N, K, vec_store, s);
    default: return launch_tile<128, 128, Epi>(A, W, epi, M, N, K, vec_store, s);
  }
}

std::string gemm_i8_kernel_name(int M, int N, int K, bool int8_out) {
  (void)K;
  const TileCand& t = kTiles[select_tile(M, N)];
  return "gemm_i8_kernel<" + std::to_string(t.bm) + "," + std::to_string(t.bn) + "," +
         (int8_out ? "EpiI8" : "EpiI32") + ">";
}

int gemm_i8_i32o(const int8_t* A, const int8_t* W, int32_t* C, int M, int N, int K,
                 hipStream_t s) {
  return dispatch(A, W, EpiI32{C}, M, N, K, C, s);
}

int gemm_i8_i8o(const int8_t* A, const int8_t* W, int8_t* C, int M, int N, int K, float alpha,
                hipStream_t s) {
  return dispatch(A, W, EpiI8{C, alpha}, M, N, K, C, s);
}

}  // namespace lsh
