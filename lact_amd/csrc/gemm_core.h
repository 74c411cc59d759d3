// Block-level GEMM main loop for gfx950: LDS-staged operand tiles, 32x32 MFMA tiles per wave,
// fp32 accumulation.  One main loop serves every contraction of the TTT operation; kernels differ
// only in which operands they chain into which accumulators and in their epilogues.
//
//   acc[m][n] += sum_k A(m,k) * B(n,k)
//
// Each operand is described independently as "K-contiguous" (element (r,k) at base[r*ld + k]) or
// "K-strided" (element (r,k) at base[k*ld + r]); K-strided bf16 tiles are pair-interleaved on the
// way into LDS so that a lane still fetches its 8 consecutive k values with 32-bit LDS reads.
//
// MFMA operands are swapped (the B tile is passed as the instruction's first operand), so each lane
// ends up owning 4 consecutive n for one m: epilogues store 8- or 16-byte vectors along n.
#pragma once
#include "common.h"

namespace lact {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_>
struct TileShape {
  static constexpr int BM = BM_, BN = BN_;
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int THREADS = 64 * WAVES_M * WAVES_N;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA tile");
};

constexpr int cmax(int a, int b) { return a > b ? a : b; }

// ------------------------------------------------------------------------------------------------
// operand tiles
// ------------------------------------------------------------------------------------------------
template <typename T, int ROWS, bool KC, int THREADS> struct OperandTile;

// bf16, K-contiguous source.  LDS: [row][BK + 8] halves.
template <int ROWS, int THREADS>
struct OperandTile<uint16_t, ROWS, true, THREADS> {
  static constexpr int BK = 32, KSTEPS = 2;
  static constexpr int LDT = BK + 8;
  static constexpr int BYTES = ROWS * LDT * 2;
  static constexpr int VPR = BK / 8, NVEC = ROWS * VPR, PER = (NVEC + THREADS - 1) / THREADS;
  typedef bf16x8 Frag;
  struct Regs { uint4 v[PER]; };

  __device__ static __forceinline__ void gload(Regs& r, const uint16_t* base, int ld, int rows_valid, int k0, int K) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int id = threadIdx.x + i * THREADS;
      const int row = id / VPR, k = k0 + (id % VPR) * 8;
      const bool p = (NVEC % THREADS == 0 || id < NVEC) && row < rows_valid && k < K;
      r.v[i] = p ? *reinterpret_cast<const uint4*>(base + (size_t)row * ld + k) : make_uint4(0, 0, 0, 0);
    }
  }
  __device__ static __forceinline__ void sstore(const Regs& r, char* smem) {
    uint16_t* t = reinterpret_cast<uint16_t*>(smem);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int id = threadIdx.x + i * THREADS;
      if (NVEC % THREADS == 0 || id < NVEC)
        *reinterpret_cast<uint4*>(t + (id / VPR) * LDT + (id % VPR) * 8) = r.v[i];
    }
  }
  __device__ static __forceinline__ Frag fetch(const char* smem, int row0, int ks, int lane) {
    const uint16_t* t = reinterpret_cast<const uint16_t*>(smem);
    const uint4 u = *reinterpret_cast<const uint4*>(t + (row0 + (lane & 31)) * LDT + ks * 16 + 8 * (lane >> 5));
    return __builtin_bit_cast(Frag, u);
  }
};

// bf16, K-strided source.  LDS: [k/2][ROWS + 8] 32-bit words, each word = (k even, k odd) of one row.
template <int ROWS, int THREADS>
struct OperandTile<uint16_t, ROWS, false, THREADS> {
  static constexpr int BK = 32, KSTEPS = 2;
  static constexpr int LDW = ROWS + 8;
  static constexpr int BYTES = (BK / 2) * LDW * 4;
  static constexpr int RG = ROWS / 8, NITEM = (BK / 2) * RG, PER = (NITEM + THREADS - 1) / THREADS;
  typedef bf16x8 Frag;
  struct Regs { uint4 lo[PER], hi[PER]; };

  __device__ static __forceinline__ void gload(Regs& r, const uint16_t* base, int ld, int rows_valid, int k0, int K) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int id = threadIdx.x + i * THREADS;
      const int k = k0 + 2 * (id / RG), r0 = (id % RG) * 8;
      const bool p = (NITEM % THREADS == 0 || id < NITEM) && r0 < rows_valid;
      const uint16_t* src = base + (size_t)k * ld + r0;
      r.lo[i] = (p && k < K) ? *reinterpret_cast<const uint4*>(src) : make_uint4(0, 0, 0, 0);
      r.hi[i] = (p && k + 1 < K) ? *reinterpret_cast<const uint4*>(src + ld) : make_uint4(0, 0, 0, 0);
    }
  }
  __device__ static __forceinline__ void sstore(const Regs& r, char* smem) {
    uint32_t* t = reinterpret_cast<uint32_t*>(smem);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int id = threadIdx.x + i * THREADS;
      if (NITEM % THREADS == 0 || id < NITEM) {
        const uint4 lo = r.lo[i], hi = r.hi[i];
        uint4 a, b;
        a.x = (lo.x & 0xffffu) | (hi.x << 16);
        a.y = (lo.x >> 16) | (hi.x & 0xffff0000u);
        a.z = (lo.y & 0xffffu) | (hi.y << 16);
        a.w = (lo.y >> 16) | (hi.y & 0xffff0000u);
        b.x = (lo.z & 0xffffu) | (hi.z << 16);
        b.y = (lo.z >> 16) | (hi.z & 0xffff0000u);
        b.z = (lo.w & 0xffffu) | (hi.w << 16);
        b.w = (lo.w >> 16) | (hi.w & 0xffff0000u);
        uint32_t* dst = t + (id / RG) * LDW + (id % RG) * 8;
        *reinterpret_cast<uint4*>(dst) = a;
        *reinterpret_cast<uint4*>(dst + 4) = b;
      }
    }
  }
  __device__ static __forceinline__ Frag fetch(const char* smem, int row0, int ks, int lane) {
    const uint32_t* t = reinterpret_cast<const uint32_t*>(smem) + (ks * 8 + 4 * (lane >> 5)) * LDW + row0 + (lane & 31);
    uint4 u;
    u.x = t[0];
    u.y = t[LDW];
    u.z = t[2 * LDW];
    u.w = t[3 * LDW];
    return __builtin_bit_cast(Frag, u);
  }
};

// fp32 tiles.  LDS: [k][ROWS + 32] floats for either source layout.
template <int ROWS, bool KC, int THREADS>
struct OperandTile<float, ROWS, KC, THREADS> {
  static constexpr int BK = 16, KSTEPS = 8;
  static constexpr int LDT = ROWS + 32;
  static constexpr int BYTES = BK * LDT * 4;
  static constexpr int NVEC = ROWS * BK / 4, PER = (NVEC + THREADS - 1) / THREADS;
  typedef float Frag;
  struct Regs { float4 v[PER]; };

  __device__ static __forceinline__ void gload(Regs& r, const float* base, int ld, int rows_valid, int k0, int K) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int id = threadIdx.x + i * THREADS;
      bool p = (NVEC % THREADS == 0 || id < NVEC);
      const float* src;
      if (KC) {
        const int row = id / (BK / 4), k = k0 + (id % (BK / 4)) * 4;
        p = p && row < rows_valid && k < K;
        src = base + (size_t)row * ld + k;
      } else {
        const int k = k0 + id / (ROWS / 4), r0 = (id % (ROWS / 4)) * 4;
        p = p && r0 < rows_valid && k < K;
        src = base + (size_t)k * ld + r0;
      }
      r.v[i] = p ? *reinterpret_cast<const float4*>(src) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  __device__ static __forceinline__ void sstore(const Regs& r, char* smem) {
    float* t = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int id = threadIdx.x + i * THREADS;
      if (NVEC % THREADS == 0 || id < NVEC) {
        if (KC) {
          const int row = id / (BK / 4), kk = (id % (BK / 4)) * 4;
          t[(kk + 0) * LDT + row] = r.v[i].x;
          t[(kk + 1) * LDT + row] = r.v[i].y;
          t[(kk + 2) * LDT + row] = r.v[i].z;
          t[(kk + 3) * LDT + row] = r.v[i].w;
        } else {
          *reinterpret_cast<float4*>(t + (id / (ROWS / 4)) * LDT + (id % (ROWS / 4)) * 4) = r.v[i];
        }
      }
    }
  }
  __device__ static __forceinline__ Frag fetch(const char* smem, int row0, int ks, int lane) {
    return reinterpret_cast<const float*>(smem)[(ks * 2 + (lane >> 5)) * LDT + row0 + (lane & 31)];
  }
};

__device__ __forceinline__ f32x16 mma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mma32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// LDS bytes a kernel built on TileShape TS needs for element type T (two stages, either layout).
template <typename T, class TS>
struct GemmSmem {
  static constexpr int A = cmax(OperandTile<T, TS::BM, true, TS::THREADS>::BYTES, OperandTile<T, TS::BM, false, TS::THREADS>::BYTES);
  static constexpr int B = cmax(OperandTile<T, TS::BN, true, TS::THREADS>::BYTES, OperandTile<T, TS::BN, false, TS::THREADS>::BYTES);
  static constexpr int BYTES = 2 * (A + B);
};

template <class TS>
__device__ __forceinline__ void zero_acc(f32x16 (&acc)[TS::TM][TS::TN]) {
#pragma unroll
  for (int i = 0; i < TS::TM; ++i)
#pragma unroll
    for (int j = 0; j < TS::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
}

// A, B point at the first row of this block's tile (K-contiguous: base + row0*ld, K-strided: base + row0).
// a_rows / b_rows: valid rows from there on (may exceed the tile).  All threads of the block must call.
template <typename T, class TS, bool A_KC, bool B_KC>
__device__ __forceinline__ void gemm_mainloop(f32x16 (&acc)[TS::TM][TS::TN], const T* __restrict__ A, int lda, int a_rows,
                                              const T* __restrict__ B, int ldb, int b_rows, int K, char* smem) {
  using TA = OperandTile<T, TS::BM, A_KC, TS::THREADS>;
  using TB = OperandTile<T, TS::BN, B_KC, TS::THREADS>;
  constexpr int BK = TA::BK;
  constexpr int STAGE = TA::BYTES + TB::BYTES;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm0 = (wave / TS::WAVES_N) * TS::WM, wn0 = (wave % TS::WAVES_N) * TS::WN;
  const int nk = (K + BK - 1) / BK;

  typename TA::Regs ra;
  typename TB::Regs rb;
  TA::gload(ra, A, lda, a_rows, 0, K);
  TB::gload(rb, B, ldb, b_rows, 0, K);
  TA::sstore(ra, smem);
  TB::sstore(rb, smem + TA::BYTES);
  __syncthreads();
  int cur = 0;
  for (int kt = 0; kt < nk; ++kt) {
    const char* sa = smem + cur * STAGE;
    const char* sb = sa + TA::BYTES;
    const bool has_next = kt + 1 < nk;
    if (has_next) {
      TA::gload(ra, A, lda, a_rows, (kt + 1) * BK, K);
      TB::gload(rb, B, ldb, b_rows, (kt + 1) * BK, K);
    }
#pragma unroll
    for (int ks = 0; ks < TA::KSTEPS; ++ks) {
      typename TA::Frag fa[TS::TM];
      typename TB::Frag fb[TS::TN];
#pragma unroll
      for (int i = 0; i < TS::TM; ++i) fa[i] = TA::fetch(sa, wm0 + i * 32, ks, lane);
#pragma unroll
      for (int j = 0; j < TS::TN; ++j) fb[j] = TB::fetch(sb, wn0 + j * 32, ks, lane);
#pragma unroll
      for (int i = 0; i < TS::TM; ++i)
#pragma unroll
        for (int j = 0; j < TS::TN; ++j) acc[i][j] = mma32(fb[j], fa[i], acc[i][j]);
    }
    if (has_next) {
      char* na = smem + (cur ^ 1) * STAGE;
      TA::sstore(ra, na);
      TB::sstore(rb, na + TA::BYTES);
    }
    __syncthreads();
    cur ^= 1;
  }
}

// Epilogue iteration.  Inside the body:  tm, tn, g index the fragment; `m`, `n` are block-local
// coordinates of 4 consecutive n; the values are acc[tm][tn][4*g + j], j = 0..3.
#define LACT_FOR_QUADS(TS)                                                                     \
  _Pragma("unroll") for (int tm = 0; tm < TS::TM; ++tm)                                        \
  _Pragma("unroll") for (int tn = 0; tn < TS::TN; ++tn)                                        \
  _Pragma("unroll") for (int g = 0; g < 4; ++g)

template <class TS> __device__ __forceinline__ int quad_m(int tm) {
  return ((threadIdx.x >> 6) / TS::WAVES_N) * TS::WM + tm * 32 + (threadIdx.x & 31);
}
template <class TS> __device__ __forceinline__ int quad_n(int tn, int g) {
  return ((threadIdx.x >> 6) % TS::WAVES_N) * TS::WN + tn * 32 + 8 * g + 4 * ((threadIdx.x & 63) >> 5);
}

}  // namespace lact
