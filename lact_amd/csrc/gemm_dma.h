// bf16 GEMM main loop for gfx950 with asynchronous global->LDS copies and a multi-stage ring.
//
//   for every phase p:   acc[p][j] += A_p (BM x K_p)  *  B_pj (BN x K_p)^T        j < NB
//
// Every operand is K-contiguous (element (r,k) at base[r*ld + k]).  A block is 4 waves; BK = 64.
// One stage of the ring holds the A tile and up to NB B tiles of one K-step; tiles are copied with
// global_load_lds_dwordx4 (16 bytes per lane straight into LDS, no VGPR staging), so STAGES-1 K-steps
// of loads stay in flight across the MFMA work -- what hides the ~1.5 us memory latency that a
// register-staged, one-step-ahead prefetch leaves exposed.  All phases run through one flat
// iteration space, so the ring never drains between phases.
//
// LDS tile layout: [row][64 bf16] = 128 B per row, unpadded (a wave's 64 lanes x 16 B land as one
// contiguous 1 KiB, 8 rows).  The 16-byte k-granule j of row r is stored at slot j ^ ((r >> 1) & 7):
// ds_read_b128 serves 16 lanes per clock, and 16 consecutive rows then cover all 64 banks.
#pragma once
#include "gemm_core.h"

// Optional in-kernel timestamps (defined only by timing experiments; expands to nothing in the library).
#ifndef LACT_TS
#define LACT_TS(i)
#endif

namespace lact {

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// 16 bytes per lane from global memory (uniform 64-bit base + per-lane 32-bit byte offset) to LDS: lane i
// lands at lds_base + 16*i (lds_base wave-uniform).  No vector-ALU work per copy: bases live in SGPRs.
// SC1: device-scope load -- always misses the vector L1 and is served by the L2.  Used where the data was written
// by another compute unit during this same kernel (the L1 is not coherent with other units' stores).
template <bool SC1 = false>
__device__ __forceinline__ void dma16(const void* sbase, uint32_t voff, uint32_t lds_base) {
  if (SC1)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 sc1\n\t" ::"s"(lds_base), "v"(voff), "s"(sbase)
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t" ::"s"(lds_base), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// K-contiguous operand: element (r, k) at base[r*ld + k].  K-strided (ks): element (r, k) at base[k*ld + r].
struct DmaOperand {
  const uint16_t* base;  // first row (r = 0, k = 0) of this block's tile
  int ld;
  int rows;              // valid rows from base on (may exceed the tile); multiple of 8 when ks
  int ks;
  int ktail = 0;         // K-strided only: valid k rows of the last K-step when K is not a multiple of 64 (0: all 64)
};

// One phase: acc[j] += A * B_j^T over K, j < nb.
template <int NBMAX>
struct DmaPhase {
  DmaOperand a;
  DmaOperand b[NBMAX];
  int nb;
  int K;
};

constexpr int DMA_BK = 64;

// Loader-wave addressing of one operand tile: the loader copies the whole tile, 8 rows (1 KiB) per
// instruction.  Rows past the operand are clamped to its last row: what they bring in only reaches output
// rows/columns that are never stored.  K must be a multiple of 64 (the host routes other shapes to the
// generic kernels).
// K-strided tiles are copied as they lie in memory, [64 k][ROWS] with the 16-byte granules of k-row k rotated
// by 4*(k % 4) positions, and read back with ds_read_b64_tr_b16: inside each group of 16 lanes, lane i
// receives element (i & 3) of the 8 bytes addressed by lanes 4j + (i >> 2), j = 0..3 -- i.e. a 4(k) x 16(r)
// patch comes back transposed, 4 consecutive k of one r per lane.  The rotation makes the four k-rows of a
// patch land in different bank groups.
constexpr int DMA_LOADERS = 4;     // loader waves per block
template <int ROWS>
struct DmaLane {
  static constexpr int NALL = ROWS / 8;            // copies per K-step, all loader waves together
  static constexpr int N = NALL / DMA_LOADERS;     // copies per K-step of this wave: copy lw, lw + DMA_LOADERS, ...
  static constexpr int G = ROWS / 8;               // granules per k-row of a K-strided tile
  static_assert(NALL % DMA_LOADERS == 0, "tile rows must split evenly over the loader waves");
  const uint16_t* base;                 // uniform
  size_t kstride;                       // uniform: elements between K-steps
  uint32_t voff[N];                     // byte offset of this lane's granule from base at K-step 0
  __device__ __forceinline__ void init(const DmaOperand& op, int lw) {
    const int lane = threadIdx.x & 63;
    base = op.base;
    kstride = op.ks ? (size_t)DMA_BK * op.ld : (size_t)DMA_BK;
#pragma unroll
    for (int ii = 0; ii < N; ++ii) {
      const int i = lw + ii * DMA_LOADERS;
      if (op.ks) {
        const int L = i * 64 + lane, k = L / G, p = L % G;
        int g = (p + G - (4 * (k & 3)) % G) % G;
        g = min(g, op.rows / 8 - 1);
        voff[ii] = (uint32_t)(((size_t)k * op.ld + g * 8) * 2);
      } else {
        const int row = i * 8 + (lane >> 3);
        const int kv = ((lane & 7) ^ ((row >> 1) & 7)) * 8;
        const int r = min(row, op.rows - 1);
        voff[ii] = (uint32_t)(((size_t)r * op.ld + kv) * 2);
      }
    }
  }
  // lds_tile: LDS address of the tile plus lw * 1024
  template <bool SC1>
  __device__ __forceinline__ void issue(int kt, uint32_t lds_tile) const {
    const uint16_t* b = base + kt * kstride;
#pragma unroll
    for (int ii = 0; ii < N; ++ii) dma16<SC1>(b, voff[ii], lds_tile + ii * DMA_LOADERS * 1024);
  }
  // The last K-step of a K-strided operand whose K ends inside it (op.ktail valid k rows): the k rows past the end
  // are read from the last valid one instead -- never past the operand.  Offsets computed here, once per phase.
  template <bool SC1>
  __device__ __forceinline__ void issue_tail(int kt, uint32_t lds_tile, const DmaOperand& op, int lw) const {
    const int lane = threadIdx.x & 63;
    const uint16_t* b = base + kt * kstride;
#pragma unroll
    for (int ii = 0; ii < N; ++ii) {
      const int L = (lw + ii * DMA_LOADERS) * 64 + lane, k = min(L / G, op.ktail - 1), p = L % G;
      int g = (p + G - (4 * ((L / G) & 3)) % G) % G;
      g = min(g, op.rows / 8 - 1);
      dma16<SC1>(b, (uint32_t)(((size_t)k * op.ld + g * 8) * 2), lds_tile + ii * DMA_LOADERS * 1024);
    }
  }
  // The k rows past the end of K in the K-strided tile that has landed at `tile` (LDS; ktail valid k rows): cleared,
  // so that whatever the other operand holds there adds nothing.  Every wave clears inside the chunks it copied
  // itself (it has waited for exactly those).
  __device__ static __forceinline__ void clear_tail(char* tile, int lw, int ktail) {
    const int lane = threadIdx.x & 63;
    const int first = ktail * ROWS * 2;   // first byte of the tile that lies past the end of K
#pragma unroll
    for (int ii = 0; ii < N; ++ii) {
      const int off = (lw + ii * DMA_LOADERS) * 1024 + lane * 16;
      if (off >= first) *reinterpret_cast<uint4*>(tile + off) = make_uint4(0, 0, 0, 0);
    }
  }
};

__device__ __forceinline__ bf16x8 dma_fetch(const char* tile, int row, int kvec) {
  const uint4 u = *reinterpret_cast<const uint4*>(tile + row * 128 + ((kvec ^ ((row >> 1) & 7)) << 4));
  return __builtin_bit_cast(bf16x8, u);
}

// ---- block -> tile mapping, aware of the 8 accelerator dies (XCDs) ----------------------------------
// The workgroups of a 1-D grid are dealt to the 8 XCDs round-robin by linear id, and every XCD has its own
// L2.  Blocks that read the same operands are therefore given ids that are congruent mod 8 and adjacent in
// that XCD's order, so that the shared tiles are fetched from HBM once and not once per die.  A group is
// one batch entry with all its tiles (batch count a multiple of 8) or one row of tiles of a batch entry.
// Only the speed depends on the dealing order, never the result.
struct TileMap {
  int gx, gy, gz;   // tiles along x and y, batch entries
  int by_batch;     // 1: group = batch entry (gx*gy members); 0: group = (batch entry, x tile) (gy members)
  __host__ __device__ int group_size() const { return by_batch ? gx * gy : gy; }
  __host__ __device__ int groups() const { return by_batch ? gz : gz * gx; }
  __host__ __device__ int grid() const { return 8 * ((groups() + 7) / 8) * group_size(); }
  __host__ __device__ bool locate_host(int L, int& x, int& y, int& z) const {   // same arithmetic, callable from host tests
    const int gs = group_size();
    const int j = L >> 3;
    const int g = (L & 7) + 8 * (j / gs), m = j % gs;
    if (g >= groups()) return false;
    if (by_batch) { z = g; x = m / gy; y = m % gy; }
    else { z = g / gx; x = g % gx; y = m; }
    return true;
  }
  __device__ __forceinline__ bool locate(int L, int& x, int& y, int& z) const { return locate_host(L, x, y, z); }
};
inline TileMap make_tile_map(int gx, int gy, int gz) {
  TileMap m;
  m.gx = gx; m.gy = gy; m.gz = gz;
  m.by_batch = gz % 8 == 0;
  return m;
}

// Fragment source of one 32-row MFMA tile: K-contiguous (one ds_read_b128) or K-strided (two transposing reads).
typedef short s16x4 __attribute__((ext_vector_type(4)));
template <int ROWS, bool KS>
struct FragSrc {
  uint32_t off0, off1;   // per-lane byte offsets at sub-step 0
  __device__ __forceinline__ void init(int row0) {   // row0: first row of the 32-row tile inside the operand tile
    const int l = threadIdx.x & 63;
    if (KS) {
      constexpr int G = ROWS / 8, RB = ROWS * 2;
      const int r = row0 + 16 * ((l >> 4) & 1) + 4 * (l & 3);
      const int p = (r / 8 + (4 * ((l >> 2) & 3)) % G) % G;
      const int krow = 8 * (l >> 5) + ((l & 15) >> 2);
      off0 = krow * RB + p * 16 + (l & 1) * 8;
      off1 = off0 + 4 * RB;
    } else {
      const int row = row0 + (l & 31);
      off0 = row * 128;
      off1 = (uint32_t)(((row >> 1) & 7) << 4 | (l >> 5) << 16);   // swizzle key and lane half, unpacked in fetch
    }
  }
  __device__ __forceinline__ bf16x8 fetch(const char* tile, int ks) const {
    if (KS) {
      constexpr int RB = ROWS * 2;
      typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
      const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off0 + ks * 16 * RB));
      const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off1 + ks * 16 * RB));
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      const s16x8 v = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
      return __builtin_bit_cast(bf16x8, v);
    } else {
      const int kvec = ks * 2 + (off1 >> 16);
      const uint4 u = *reinterpret_cast<const uint4*>(tile + off0 + (((kvec << 4) ^ (off1 & 0xffff))));
      return __builtin_bit_cast(bf16x8, u);
    }
  }
};

// Scheduling directive: MFMAS matrix instructions with READS LDS reads spread behind the first of them.
template <int READS, int MFMAS, int I = 0>
__device__ __forceinline__ void sched_interleave() {
  if constexpr (I < MFMAS) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    constexpr int RPM = (READS + MFMAS - 1) / MFMAS;
    constexpr int left = READS - I * RPM;
    if constexpr (left > 0) __builtin_amdgcn_sched_group_barrier(0x100, left < RPM ? left : RPM, 0);
    sched_interleave<READS, MFMAS, I + 1>();
  }
}

template <class TS, int NBMAX, int STAGES>
struct DmaSmem {
  static constexpr int A_BYTES = TS::BM * 128, B_BYTES = TS::BN * 128;
  static constexpr int STAGE = A_BYTES + NBMAX * B_BYTES;
  static constexpr int BYTES = STAGE * STAGES;
  static_assert(BYTES <= 160 * 1024, "ring does not fit the 160 KiB LDS");
};

constexpr int DMA_THREADS = 256 + 64 * DMA_LOADERS;   // four MFMA waves + the loader waves

// Flat multi-phase pipeline with a dedicated loader wave.
//
// A wave that issues a vector-memory instruction while the address FIFO is full stalls in order -- its
// MFMAs stall with it -- and with four waves each copying a quarter of every tile the matrix pipe ran
// dry for as long as the copies took (measured: K-step time = MFMA time + copy time).  So wave 4 issues
// every copy (scalar bases, per-lane offsets precomputed: no vector ALU work per copy) and waves 0-3
// only read fragments and issue MFMAs.  One barrier per K-step:
//     loader:    wait until stage kt has landed; barrier; refill the stage the MFMA waves just left
//     consumers: barrier; MFMAs on stage kt
// TAILS: a K-strided A operand may end inside its last K-step (DmaOperand::ktail), together with its B operand.
template <class TS, int NBMAX, int NPH, int STAGES, bool SC1 = false, bool TAILS = false>
struct DmaPipe {
  using SM = DmaSmem<TS, NBMAX, STAGES>;
  static constexpr int loads(int nb) { return (TS::BM + nb * TS::BN) / 8; }   // loader copies per K-step

  char* smem;
  const DmaPhase<NBMAX>* ph;
  int total;

  __device__ __forceinline__ DmaPipe(char* s, const DmaPhase<NBMAX>* phases) : smem(s), ph(phases), total(0) {
#pragma unroll
    for (int i = 0; i < NPH; ++i) total += ph[i].K / DMA_BK;
  }
  __device__ static __forceinline__ bool is_loader() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) >= 4; }

  // ---- loader waves: every copy of every phase, split evenly.  MINLOADS: smallest per-K-step copy count of
  // any phase (all loader waves together).  The copy rate of a compute unit grows with the number of waves that
  // issue the copies, not only with the bytes in flight (measured with loads that hit the L2: 22 / 45 / 75 GB/s
  // per compute unit from 2 / 4 / 8 issuing waves at the same depth), so four loader waves beside the four MFMA
  // waves: eight waves are what the register budget of the MFMA waves (256 each) allows.
  template <int MINLOADS>
  __device__ __forceinline__ void load_all() {
    constexpr int PER_WAVE = MINLOADS / DMA_LOADERS;
    constexpr int AHEAD = (STAGES - 2) * PER_WAVE > 63 ? 63 : (STAGES - 2) * PER_WAVE;
    const int lw = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) - 4;
    DmaLane<TS::BM> la;
    DmaLane<TS::BN> lb[NBMAX];
    int cp = -1, ckt = 0, cnk = 0, cnb = 0, issued = 0;
    auto next_phase = [&]() {
      ++cp;
      ckt = 0;
#pragma unroll
      for (int i = 0; i < NPH; ++i)
        if (i == cp) {
          la.init(ph[i].a, lw);
#pragma unroll
          for (int j = 0; j < NBMAX; ++j) lb[j].init(ph[i].b[j], lw);
          cnb = ph[i].nb;
          cnk = ph[i].K / DMA_BK;
        }
    };
    auto issue_stage = [&]() {
      const uint32_t base = lds_addr(smem + (issued % STAGES) * SM::STAGE) + lw * 1024;
      bool tail = false;
      if constexpr (TAILS) {
        if (ckt + 1 == cnk) {
#pragma unroll
          for (int i = 0; i < NPH; ++i)
            if (i == cp && ph[i].a.ks && ph[i].a.ktail > 0) {
              tail = true;
              la.template issue_tail<SC1>(ckt, base, ph[i].a, lw);
#pragma unroll
              for (int j = 0; j < NBMAX; ++j)
                if (j < cnb) lb[j].template issue_tail<SC1>(ckt, base + SM::A_BYTES + j * SM::B_BYTES, ph[i].b[j], lw);
            }
        }
      }
      if (!tail) {
        la.template issue<SC1>(ckt, base);
#pragma unroll
        for (int j = 0; j < NBMAX; ++j)
          if (j < cnb) lb[j].template issue<SC1>(ckt, base + SM::A_BYTES + j * SM::B_BYTES);
      }
      ++issued;
      if (++ckt == cnk)
        while (cp + 1 < NPH) {
          next_phase();
          if (cnk > 0) break;
        }
    };
    do next_phase(); while (cnk == 0 && cp + 1 < NPH);
    for (int i = 0; i < STAGES - 1 && issued < total; ++i) issue_stage();
    // TAILS: the stage that holds a phase's ragged last K-step gets the k rows past the end of its A tile cleared
    // once it has landed, before the MFMA waves are let in
    int tail_step[NPH], tail_rows[NPH], acc_steps = 0;
    if constexpr (TAILS) {
#pragma unroll
      for (int i = 0; i < NPH; ++i) {
        acc_steps += ph[i].K / DMA_BK;
        tail_rows[i] = (ph[i].a.ks && ph[i].K > 0) ? ph[i].a.ktail : 0;
        tail_step[i] = acc_steps - 1;
      }
    }
    for (int kt = 0; kt < total; ++kt) {
      if (kt + STAGES - 2 < total) wait_vmcnt<AHEAD>();
      else wait_vmcnt<0>();
      if constexpr (TAILS) {
#pragma unroll
        for (int i = 0; i < NPH; ++i)
          if (tail_rows[i] > 0 && kt == tail_step[i]) DmaLane<TS::BM>::clear_tail(smem + (kt % STAGES) * SM::STAGE, lw, tail_rows[i]);
      }
      __syncthreads();
      if (issued < total) issue_stage();
    }
  }

  // ---- MFMA waves: one phase, nk K-steps into acc[0..NB).  `step` counts K-steps over all phases.
  template <int NB, bool A_KS = false, bool B_KS = false>
  __device__ __forceinline__ void run_phase(int nk, int& step, f32x16 (&acc)[NB][TS::TM][TS::TN]) {
    const int wave = threadIdx.x >> 6;
    FragSrc<TS::BM, A_KS> sa[TS::TM];
    FragSrc<TS::BN, B_KS> sb[TS::TN];
#pragma unroll
    for (int i = 0; i < TS::TM; ++i) sa[i].init((wave / TS::WAVES_N) * TS::WM + i * 32);
#pragma unroll
    for (int n = 0; n < TS::TN; ++n) sb[n].init((wave % TS::WAVES_N) * TS::WN + n * 32);
    if (nk <= 0) return;
    // Rolling fragment pipeline: the fragments of sub-step s+1 are fetched before the MFMAs of sub-step s
    // issue, across K-steps too -- the barrier that opens stage kt+1 and the fetch of its first fragments
    // sit in front of the last MFMA group of stage kt, which hides the LDS latency.
    bf16x8 fa[2][TS::TM], fb[2][NB][TS::TN];
    const char* st = nullptr;
    auto fetch = [&](int buf, int ks) {
#pragma unroll
      for (int i = 0; i < TS::TM; ++i) fa[buf][i] = sa[i].fetch(st, ks);
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int n = 0; n < TS::TN; ++n) fb[buf][j][n] = sb[n].fetch(st + SM::A_BYTES + j * SM::B_BYTES, ks);
    };
    auto mfmas = [&](int buf) {
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int i = 0; i < TS::TM; ++i)
#pragma unroll
          for (int n = 0; n < TS::TN; ++n) acc[j][i][n] = mma32(fb[buf][j][n], fa[buf][i], acc[j][i][n]);
    };
    // Instruction order within a (fetch next, MFMAs current) pair: LDS reads behind each of the first MFMAs,
    // so that the reads spread under the matrix work instead of piling up in front of a wait.
    constexpr int READS = (A_KS ? 2 : 1) * TS::TM + (B_KS ? 2 : 1) * NB * TS::TN, MFMAS = NB * TS::TM * TS::TN;
    auto interleave = [&]() {
      sched_interleave<READS, MFMAS>();
    };
    __syncthreads();
    st = smem + (step % STAGES) * SM::STAGE;
    fetch(0, 0);
    for (int kt = 0; kt < nk; ++kt) {
      fetch(1, 1);
      mfmas(0);
      interleave();
      fetch(0, 2);
      mfmas(1);
      interleave();
      fetch(1, 3);
      mfmas(0);
      interleave();
      ++step;
      if (kt + 1 < nk) {
        __syncthreads();
        st = smem + (step % STAGES) * SM::STAGE;
        fetch(0, 0);
      }
      mfmas(1);
      interleave();
    }
  }
};

// ---- epilogue staging: accumulators -> LDS tile -> whole rows ------------------------------------
// A lane owns 4 consecutive n of 32 different rows per fragment; storing that straight to memory touches
// 32 cache lines per instruction.  Staging the tile in LDS lets every store instruction cover whole rows.
// Vector-ALU work bounds this phase, so all LDS addresses are (per-thread base + compile-time offset)
// and the row loop advances pointers instead of dividing.
//
// StageTile<TS, E>: [BM][BN + PAD] elements of E bytes, 16-byte chunks; RPP rows are copied per pass.
template <class TS, int E>
struct StageTile {
  static constexpr int CH = 16 / E;                    // elements per 16-byte chunk
  static constexpr int LD = TS::BN + (E == 2 ? 8 : 4); // elements
  static constexpr int BYTES = TS::BM * LD * E;
  static constexpr int LPR = TS::BN / CH;              // lanes per row
  static constexpr int RPP = DMA_THREADS / LPR;        // rows per pass: MFMA and loader waves all copy out
  static constexpr int PASSES = (TS::BM + RPP - 1) / RPP;

  // byte offset inside the tile of this lane's first quad (fragment 0,0, g = 0)
  __device__ static __forceinline__ int lane_base() {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = (wave / TS::WAVES_N) * TS::WM + (lane & 31), n = (wave % TS::WAVES_N) * TS::WN + 4 * (lane >> 5);
    return (m * LD + n) * E;
  }
  // compile-time offset of fragment (tm, tn, g) relative to lane_base()
  __device__ static constexpr int frag_off(int tm, int tn, int g) { return (tm * 32 * LD + tn * 32 + g * 8) * E; }
  __device__ static __forceinline__ void put4(char* base, int tm, int tn, int g, float a, float b, float c, float d) {
    if (E == 2) Elem<uint16_t>::store4(reinterpret_cast<uint16_t*>(base + frag_off(tm, tn, g)), a, b, c, d);
    else *reinterpret_cast<float4*>(base + frag_off(tm, tn, g)) = make_float4(a, b, c, d);
  }
  __device__ static __forceinline__ void get4(const char* base, int tm, int tn, int g, float (&o)[4]) {
    static_assert(E == 2, "staged inputs are bf16 tiles");
    Elem<uint16_t>::load4(reinterpret_cast<const uint16_t*>(base + frag_off(tm, tn, g)), o);
  }
  // this thread's position in the copy-out phase
  __device__ static __forceinline__ bool active() { return (int)threadIdx.x < RPP * LPR; }
  __device__ static __forceinline__ int row0() { return threadIdx.x / LPR; }
  __device__ static __forceinline__ int col0() { return (threadIdx.x % LPR) * CH; }
  // 16 bytes of copy-out pass `ps` for the thread whose first row is r0 (src = its address in pass 0); a pass
  // that would leave the tile reads pass 0 again (the caller discards it)
  __device__ static __forceinline__ uint4 read16(const char* src, int r0, int ps) {
    const bool inside = (ps + 1) * RPP <= TS::BM || r0 + ps * RPP < TS::BM;
    return *reinterpret_cast<const uint4*>(src + (inside ? ps * RPP * LD * E : 0));
  }
};

// Plain copy of a staged bf16 tile to `out` (row stride ld elements), rows/cols = valid extent of the tile.
template <class TS>
__device__ __forceinline__ void copy_out_b16(const char* smem, uint16_t* out, int ld, int rows, int cols) {
  using ST = StageTile<TS, 2>;
  if (!ST::active()) return;
  const int r0 = ST::row0(), c0 = ST::col0();
  if (c0 >= cols) return;
  const char* src = smem + (r0 * ST::LD + c0) * 2;
  uint16_t* dst = out + (size_t)r0 * ld + c0;
  const size_t step = (size_t)ST::RPP * ld;
  uint4 ug[8];
#pragma unroll
  for (int ps = 0; ps < ST::PASSES; ++ps) {
    if (ps % 8 == 0) {
#pragma unroll
      for (int g = 0; g < 8; ++g)
        if (ps + g < ST::PASSES) ug[g] = ST::read16(src, r0, ps + g);
    }
    if (r0 + ps * ST::RPP < rows && r0 + ps * ST::RPP < TS::BM) *reinterpret_cast<uint4*>(dst) = ug[ps % 8];
    dst += step;
  }
}

}  // namespace lact
