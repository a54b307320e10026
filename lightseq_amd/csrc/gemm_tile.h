// Pieces of the int8 GEMM shared by the stand-alone kernels (gemm_i8.hip) and the kernels that
// run a product as one phase of a longer launch (xcd_ffn_kernels.hip): the plain int32, the
// requantising and the tabulated epilogue, and the K loop of one large output tile.
#pragma once
#include "ls_device.h"
#include "tile_common.h"

#include <type_traits>

namespace lsh {

// ---------------------------------------------------------------------------------
// Epilogues.  store16(m, n, N, c, full): c[0..15] are C[m, n .. n+15]; `full` means all
// 16 columns exist and the vector path may be used.
// ---------------------------------------------------------------------------------
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
  // one element (the decode-step kernels give every thread one element of a 16 x 16 block)
  struct Pre1 {};
  __device__ __forceinline__ Pre1 prefetch1(int) const { return Pre1{}; }
  struct Blk1 {
    int n;
  };
  __device__ __forceinline__ Blk1 block1(int n) const { return Blk1{n}; }
  __device__ __forceinline__ void store1(long m, Blk1 blk, int N, int acc, Pre1, const int8_t*,
                                         int) const {
    C[m * N + blk.n] = acc;
  }
  bool vec_ok(int N) const { return N % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0; }
  static const char* name() { return "EpiI32"; }
};

__device__ __forceinline__ void store16_i8(int8_t* p, int n, int N, const int (&q)[16], bool full) {
  if (full) {
    uint4 o;
    o.x = pack4_i8(q[0], q[1], q[2], q[3]);
    o.y = pack4_i8(q[4], q[5], q[6], q[7]);
    o.z = pack4_i8(q[8], q[9], q[10], q[11]);
    o.w = pack4_i8(q[12], q[13], q[14], q[15]);
    *reinterpret_cast<uint4*>(p) = o;
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (n + i < N) p[i] = (int8_t)q[i];
  }
}

struct EpiI8 {
  int8_t* C;
  float alpha;
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    if (full) {
      *reinterpret_cast<uint4*>(C + m * N + n) = requant16_packed(c, alpha);
      return;
    }
    int q[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) q[i] = requant_acc(c[i], alpha);
    store16_i8(C + m * N + n, n, N, q, full);
  }
  struct Pre1 {};
  __device__ __forceinline__ Pre1 prefetch1(int) const { return Pre1{}; }
  struct Blk1 {
    int n;
  };
  __device__ __forceinline__ Blk1 block1(int n) const { return Blk1{n}; }
  __device__ __forceinline__ void store1(long m, Blk1 blk, int N, int acc, Pre1, const int8_t*,
                                         int) const {
    C[m * N + blk.n] = (int8_t)requant_acc_fast(acc, alpha);
  }
  bool vec_ok(int N) const { return N % 16 == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0; }
  static const char* name() { return "EpiI8"; }
};

// The same epilogue through a table.  After the requantisation an element is one of 255
// codes, and what follows (dequantise, add the column's bias, activation, requantise)
// depends only on that code and the column: table[n][code + 128], N x 256 bytes built once
// per weight matrix by build_act_lut with the very device function EpiActI8 evaluates, so
// the result is bit-identical.  The bias + GELU arithmetic costs ~35 vector instructions per
// element -- more than the matrix cores spend on a K = 768 product -- while the lookup is
// one byte load per element from a table that stays in L2 (768 KB for N = 3072); the lanes
// of one load instruction read two table rows, i.e. a handful of cache lines.
struct EpiLutI8 {
  int8_t* C;
  const int8_t* lut;
  float alpha;
  __device__ __forceinline__ void store16(long m, int n, int N, const v16i& c, bool full) const {
    int q[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int col = n + i < N ? n + i : N - 1;
      q[i] = lut[(long)col * 256 + requant_acc(c[i], alpha) + 128];
    }
    store16_i8(C + m * N + n, n, N, q, full);
  }
  // the same with the table rows of the tile's columns staged in LDS (`tab`: 256 bytes per
  // column, first row = the tile's first column; n_local = n - first column)
  __device__ __forceinline__ void store16_lds(long m, int n, int N, const v16i& c, bool full,
                                              const int8_t* tab, int n_local) const {
    int q[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      q[i] = tab[(n_local + i) * 256 + requant_acc_fast(c[i], alpha) + 128];
    store16_i8(C + m * N + n, n, N, q, full);
  }
  // one element, the table rows of the workgroup's columns staged in LDS (n_local: the
  // element's column among them)
  struct Pre1 {};
  __device__ __forceinline__ Pre1 prefetch1(int) const { return Pre1{}; }
  struct Blk1 {
    int n;
  };
  __device__ __forceinline__ Blk1 block1(int n) const { return Blk1{n}; }
  __device__ __forceinline__ void store1(long m, Blk1 blk, int N, int acc, Pre1,
                                         const int8_t* tab, int n_local) const {
    C[m * N + blk.n] = tab[n_local * 256 + requant_acc_fast(acc, alpha) + 128];
  }
  bool vec_ok(int N) const { return N % 16 == 0 && (reinterpret_cast<uintptr_t>(C) & 15u) == 0; }
  static const char* name() { return "EpiLutI8"; }
};

template <typename Epi>
__device__ __forceinline__ const int8_t* epi_lut(const Epi&) { return nullptr; }
__device__ __forceinline__ const int8_t* epi_lut(const EpiLutI8& e) { return e.lut; }

// ---------------------------------------------------------------------------------
// One output tile of TM x TN = (WGM * MB * 32) x (WGN * NB * 32) on WGM * WGN wavefronts: rows
// row0 .. row0 + TM of A (clamped to row_end - 1 when read, not stored from row_end on) times
// rows tn * TN .. of W.  K steps of 128 bytes go through a ring of NST stages in `smem`
// ((TM + TN) * 128 bytes each) filled by global_load_lds_dwordx4; fragments are double-buffered
// per 32-byte slice and the issue order inside a slice is pinned (one LDS read after each of
// the first MFMAs); the step's barrier sits before the last slice's MFMAs, after it the freed
// stage is refilled with step kt + NST.  The tabulated epilogue brings its TN x 256-byte table
// into the stage that the second-to-last step frees, while the last step is multiplied.
// Every wavefront of the workgroup must call it (it holds workgroup barriers: tile_gemm_barriers
// of them); the caller separates two calls by a barrier of its own.
// Preconditions: K % 128 == 0, K / 128 >= NST, N % 16 == 0, 32-bit operand offsets, operands
// 16-byte aligned.  A_FROM_L2: the rows of A were written by other compute units of this XCD
// during this launch (read past the vector cache).
// ---------------------------------------------------------------------------------
template <typename Epi, int NST>
constexpr int tile_gemm_barriers(int nk) {
  return nk + (std::is_same<Epi, EpiLutI8>::value ? 1 : 0);
}

template <typename Epi, int WGM, int WGN, int MB, int NB, int NST, bool A_FROM_L2 = false>
__device__ __forceinline__ void tile_gemm(const int8_t* __restrict__ A,
                                          const int8_t* __restrict__ W, const Epi& epi, int row0,
                                          int row_end, int N, int K, int tn, int8_t* smem) {
  constexpr bool LUT = std::is_same<Epi, EpiLutI8>::value;
  // The operand order of the MFMA decides what a lane's 16 accumulators are: weight rows first,
  // 16 adjacent columns of one output row (one 16-byte store of int8 codes); activations first,
  // 16 rows of one column -- the layout for int32 output, whose stores then cover whole lines.
  constexpr bool ROWS_IN_REGS = std::is_same<Epi, EpiI32>::value;
  constexpr int NWV = WGM * WGN;
  constexpr int TM = WGM * MB * 32, TN = WGN * NB * 32;
  constexpr int STAGE = (TM + TN) * kBK;
  constexpr int NA = TM / 8 / NWV, NW = TN / 8 / NWV, PER = NA + NW;  // 1-KB loads per wavefront
  constexpr int NTAB = TN / 4 / NWV;  // table loads per wavefront
  static_assert(TM % (8 * NWV) == 0 && TN % (8 * NWV) == 0, "stage rows split over the wavefronts");
  static_assert((NST - 1) * PER < 64, "vmcnt range");
  static_assert(!LUT || (TM >= TN && TN % (4 * NWV) == 0), "table fits a freed stage");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN, l32 = lane & 31, g = lane >> 5;
  const int nk = K / kBK;

  uint32_t a_src[NA], w_src[NW];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int row = (wave + NWV * i) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ key_act(row);
    a_src[i] = (uint32_t)min(row0 + row, row_end - 1) * (uint32_t)K + c * 16;
  }
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int row = (wave + NWV * i) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ key_wgt(row);
    w_src[i] = (uint32_t)min(tn * TN + row, N - 1) * (uint32_t)K + c * 16;
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
  auto dma1 = [&](const int8_t* base, uint32_t voff, uint32_t lds) {
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff),
                 "s"(base)
                 : "memory");
  };
  // the same past this compute unit's vector cache (sc1: the line is taken from the L2), for an
  // operand that another compute unit of the XCD wrote during this launch
  auto dma1_l2 = [&](const int8_t* base, uint32_t voff, uint32_t lds) {
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 sc1" ::"s"(lds), "v"(voff),
                 "s"(base)
                 : "memory");
  };
  auto issue = [&](int kt, int slot) {  // K step kt into ring slot `slot`
    const uint32_t base = lds0 + slot * STAGE;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      if (A_FROM_L2) dma1_l2(A + kt * kBK, a_src[i], base + (wave + NWV * i) * 1024);
      else dma1(A + kt * kBK, a_src[i], base + (wave + NWV * i) * 1024);
    }
#pragma unroll
    for (int i = 0; i < NW; ++i)
      dma1(W + kt * kBK, w_src[i], base + TM * kBK + (wave + NWV * i) * 1024);
  };
  // LDS byte offset of this lane's fragment chunk for K slice 0; slice ks is at (offset ^ (ks << 5)):
  // chunk index 2 * ks + g, swizzled by the row key, and 2 * ks only touches bits 1-2 of it
  int a_base[MB], w_base[NB];
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int row = wm * (MB * 32) + i * 32 + l32;
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
  auto load_frag = [&](Frag& f, const int8_t* stage, int ks) {
#pragma unroll
    for (int i = 0; i < MB; ++i)
      f.a[i] = *reinterpret_cast<const v4i*>(stage + (a_base[i] ^ (ks << 5)));
#pragma unroll
    for (int j = 0; j < NB; ++j)
      f.w[j] = *reinterpret_cast<const v4i*>(stage + (w_base[j] ^ (ks << 5)));
  };
  v16i acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) acc[i][j] = (v16i)0;
  auto mma = [&](const Frag& f) {
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j)
        acc[i][j] = ROWS_IN_REGS
                        ? __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a[i], f.w[j], acc[i][j], 0, 0, 0)
                        : __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w[j], f.a[i], acc[i][j], 0, 0, 0);
  };
  // issue order of one slice: an LDS read of the next slice after each of the first MFMAs
  auto pattern = [&]() {
#pragma unroll
    for (int q = 0; q < MB + NB; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    if (MB * NB > MB + NB) __builtin_amdgcn_sched_group_barrier(0x008, MB * NB - (MB + NB), 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  Frag f[2];
  auto slices = [&](const int8_t* stage) {  // slices 1..3 read, slices 0..2 multiplied
#pragma unroll
    for (int ks = 1; ks < 4; ++ks) {
      load_frag(f[ks & 1], stage, ks);
      mma(f[(ks - 1) & 1]);
      pattern();
    }
  };

#pragma unroll
  for (int s = 0; s < NST; ++s) issue(s, s);
  wait_vmcnt<(NST - 1) * PER>();
  __builtin_amdgcn_s_barrier();
  load_frag(f[0], smem, 0);
  int slot = 0;
  // steady state: a step ends by refilling its own slot with step kt + NST
  for (int kt = 0; kt < nk - NST; ++kt) {
    slices(smem + slot * STAGE);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront has read all of the stage
    wait_vmcnt<(NST - 2) * PER>();       // its own loads of step kt + 1 have landed ...
    __builtin_amdgcn_s_barrier();        // ... and everyone's; everyone is done with step kt
    issue(kt + NST, slot);
    __builtin_amdgcn_sched_barrier(0);
    if (++slot == NST) slot = 0;
    load_frag(f[0], smem + slot * STAGE, 0);
    mma(f[1]);
    pattern();
  }
  // drain: NST - 1 steps without a refill, then the last step
  int tab_slot = 0;
#pragma unroll
  for (int t = 0; t < NST - 1; ++t) {
    slices(smem + slot * STAGE);
    __builtin_amdgcn_s_waitcnt(0xC07F);
    if (NST - 2 - t == 0) wait_vmcnt<0>();
    else if (NST - 2 - t == 1) wait_vmcnt<PER>();
    else wait_vmcnt<2 * PER>();
    __builtin_amdgcn_s_barrier();
    if (LUT && t == NST - 2) {
      // the slot of the second-to-last step is free: the tile's table rows go there
      tab_slot = slot;
      const long first = (long)tn * TN * 256, last = (long)N * 256 - 16;
#pragma unroll
      for (int i = 0; i < NTAB; ++i) {
        const int q = wave + NWV * i;
        const long off = min(first + q * 1024 + lane * 16, last);  // rows beyond N: never stored
        dma1(reinterpret_cast<const int8_t*>(epi_lut(epi)), (uint32_t)off,
             lds0 + slot * STAGE + q * 1024);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (++slot == NST) slot = 0;
    load_frag(f[0], smem + slot * STAGE, 0);
    mma(f[1]);
    pattern();
  }
  slices(smem + slot * STAGE);
  mma(f[1]);
  if (LUT) {
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
  }
  if constexpr (ROWS_IN_REGS) {
    // int32 output: a lane holds column sigma(l32) of its block and the rows 8 (k / 4) + 4 g +
    // k % 4 in register k, so a store instruction writes two whole 128-byte lines (32 lanes, 32
    // adjacent columns of one row each)
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int n = tn * TN + wn * (NB * 32) + j * 32 + sigma(l32);
        int32_t* cp = epi.C + n;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          const long m = (long)row0 + wm * (MB * 32) + i * 32 + 8 * (k >> 2) + 4 * g + (k & 3);
          if (m < row_end && n < N) cp[m * N] = acc[i][j][k];
        }
      }
    return;
  }
  const int8_t* tab = smem + tab_slot * STAGE;
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const long m = (long)row0 + wm * (MB * 32) + i * 32 + l32;
    if (m < row_end) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int nl = wn * (NB * 32) + j * 32 + 16 * g;
        const int n = tn * TN + nl;
        if (n < N) {
          if constexpr (LUT) epi.store16_lds(m, n, N, acc[i][j], true, tab, nl);
          else epi.store16(m, n, N, acc[i][j], true);
        }
      }
    }
  }
}

}  // namespace lsh
