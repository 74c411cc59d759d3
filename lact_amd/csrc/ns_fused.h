// Newton-Schulz iterations (forward, and their backward) as ONE launch per batch of matrices.
//
// The unfused path runs three dependent GEMM kernels per iteration over 48 small matrices: 6 K-steps of
// matrix work per block between a launch gap and a cache write-back, 30 launches per update step.  Here the
// blocks that own the tiles of one matrix stay resident, run the stages back to back and meet at a barrier
// of their own between stages:
//
//   * the block -> tile map gives all tiles of a matrix linear ids that are congruent mod 8, i.e. the same
//     XCD (workgroups are dealt to the 8 XCDs round-robin), so everything the group exchanges lives in one L2;
//   * a stage's stores are complete in that L2 once the block has waited for them (vmcnt) -- no L2
//     write-back is needed inside an XCD -- and the operands written by the partner blocks are read with
//     device-scope loads that miss the (non-coherent) vector L1;
//   * the barrier is a counter in that L2: arrive = atomic add, wait = poll (measured ~1.3 us per barrier
//     against ~4.5 us of launch gap plus the write-back of everything the kernel stored).
//
// Should the hardware place a group's blocks on different XCDs (each block publishes its XCC id at the
// start and the group checks), the group falls back to device-scope release/acquire fences around every
// barrier -- correct anywhere, only slower.  Every poll loop is bounded: on a timeout the block raises
// the error word and moves on, so that all waves always exit.
//
// Deadlock freedom needs each group to become resident as a whole.  The host launches at most 256 blocks
// (one per compute unit at this LDS size) per kernel and orders fused launches of one process after each
// other with an event, so two such kernels never hold compute units while waiting for each other.
#pragma once
#include "gemm_dma_kernels.h"
#include "state_kernels.h"

// Optional in-kernel timestamps (defined only by timing experiments; expands to nothing in the library).
#ifndef LACT_NS_TS
#define LACT_NS_TS(i)
#endif

namespace lact {

constexpr int NS_FUSED_MAX_STEPS = 8;
constexpr long long NS_FUSED_SPIN_LIMIT = 4000000;   // default bound of a barrier wait, in polls of ~64 clocks: a fraction of a second

struct NsFusedParams {
  int n, z0;                 // matrices of this launch: global indices z0 .. z0+n-1 of the packed [3b] arrays
  int r, c, S;               // Newton-Schulz orientation [r, c], r <= c, both multiples of the tile edge; iterations
  int nb, mask, plain;       // u_out is written transposed for matrices whose (z / nb) bit of mask is set
  float coeffs[3 * NS_FUSED_MAX_STEPS];
  // forward:  X_0 in xf[0] (fp32) and xb (bf16);  saves X_k, A_k, B_k (bf16) per iteration
  float* xf[2];
  uint16_t* xb; long long xb_it_stride;            // X_k at xb + k * xb_it_stride, k < S
  uint16_t* ab; uint16_t* bb; long long sq_it_stride;
  uint16_t* cab;                                   // forward: c * A of the running iteration (one [r, r] buffer per matrix)
  float* u_out;                                    // X_S, fp32, original orientation
  // backward: incoming gradient in gxf[0] / gxb[0]; the result ends in gxf[S & 1]
  float* gxf[2]; uint16_t* gxb[2]; uint16_t* sg; uint16_t* gas;
  // forward, optional first stage: X_0 = G / (|G|_F + 1e-7) from the bf16 gradient g16 (laid out like xb) and the
  // partial sums of its squares; writes xf[0], xb (iteration 0) and the norms.  Null g16: X_0 is there already.
  const uint16_t* g16; const float* ss_part; int nparts, part0, part1;   // partial rows part0 + z and (if >= 0) part1 + z
  float* norms;              // [n] of this batch
  // backward, optional last stages (the backward of that normalisation): every block writes <G_final, g16> over
  // its tile to dot_part[z][member]; with gc set, the blocks then meet once more and each writes its tile of
  //   gc = G_final / (n + 1e-7) - g16 * <G_final, g16> / (n (n + 1e-7)^2)
  // (the gradient w.r.t. the Newton-Schulz input in the compute type; norms as written by the forward)
  float* dot_part; uint16_t* gc;
  // with gc and a momentum state in the program: the gradient that arrives at the state after this update is added
  // (carry_valid), the one for the state before it is written back (carry_write: g * mbar), and the partial dots
  // <g, M_prev> over this block's tile go to mdot_part[z][member] (m_prev set).  All arrays packed like gc.
  float* gm_carry; int carry_valid, carry_write;
  const float* m_prev; const float* mbar; float* mdot_part;
  unsigned* sync;            // [n][32] words, zeroed before the launch: word 0 = arrivals, word 1 = XCC id mask
  unsigned* error;           // set to 1 by a block whose barrier timed out
  unsigned* sticky;          // per-device count of such time-outs (not cleared between calls), or null
  long long spin_limit;      // polls a block waits at a barrier before it gives up
};

struct GroupBarrier {
  unsigned* ctr;
  unsigned* sticky;          // per-device count of timed-out waits, never cleared by a kernel (lact_check_async_error reads it)
  unsigned members, epoch;
  long long limit;
  bool split;                // group spread over several XCDs: fence at device scope
  __device__ __forceinline__ void init(unsigned* line, unsigned nmembers, unsigned* error, long long spin_limit, unsigned* sticky_count) {
    ctr = line; members = nmembers; epoch = 0; split = false; limit = spin_limit; sticky = sticky_count;
    unsigned xcc = 0;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    if (threadIdx.x == 0) __hip_atomic_fetch_or(line + 1, 1u << (xcc & 0xf), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sync(error, true);
    unsigned m = __hip_atomic_load(line + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    split = (m & (m - 1)) != 0;
  }
  // all threads of the block call it
  __device__ __forceinline__ void sync(unsigned* error, bool heavy = false) {
    // Every wave waits for its own stores of the stage: a store that has been waited for is in this XCD's L2 (the
    // vector L1 writes through), which is where the partner blocks' device-scope loads look.  Without the wait the
    // arrival below could overtake a store that is still on its way to another L2 channel.
    wait_vmcnt<0>();
    __syncthreads();
    if (threadIdx.x == 0) {
      const bool fence = heavy || split;
      if (fence) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const unsigned target = members * (++epoch);
      long long spins = 0;
      while (__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
        __builtin_amdgcn_s_sleep(1);
        if (++spins > limit) {
          __hip_atomic_store(error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (sticky) __hip_atomic_fetch_add(sticky, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
      }
      if (fence) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    } else {
      ++epoch;
    }
    __syncthreads();
  }
};

template <int NT>
__device__ __forceinline__ RowGemmDmaParams<NT> ns_row_params() {
  RowGemmDmaParams<NT> q;
  q.g.accumulate = 0; q.g.aux = nullptr; q.g.ldaux = 0; q.g.bsaux = 0; q.g.alpha = 1.f; q.g.beta = 0.f;
  q.g.out_c = nullptr; q.g.out_t = nullptr; q.g.transpose_mask = 0; q.g.nb = 1; q.g.round_out_bf16 = 0;
  q.g.out2 = nullptr; q.g.alpha2 = 0.f;
  q.out_ct = nullptr;
  return q;
}
__device__ __forceinline__ void ns_term(RowGemmTerm& t, const void* A, int lda, long long bsA, const void* B, int ldb, long long bsB, int K) {
  t.A = A; t.lda = lda; t.bsA = bsA; t.B = B; t.ldb = ldb; t.bsB = bsB; t.K = K;
}

// <gx, g16> over one TS::BM x TS::BN tile whose first element is at offset zo of both arrays (row stride c): every thread
// takes the granules of 8 elements threadIdx.x, threadIdx.x + DMA_THREADS, ... and keeps what it read (ga, gb: the fp32
// values, gi: the bf16 ones).  Returns this thread's partial sum.  The fused kernel and k_ns_bwd_dot_tiles both sum a
// tile through this one function and block_sum, so the two paths produce the same bits.
template <class TS, int NG>
__device__ __forceinline__ float ns_tile_dot(const float* gx, const uint16_t* g16, size_t zo, int c, float4 (&ga)[NG], float4 (&gb)[NG], uint4 (&gi)[NG]) {
  constexpr int GR = TS::BN / 8;
  static_assert(NG == (TS::BM * GR + DMA_THREADS - 1) / DMA_THREADS, "granules per thread");
  float dot = 0.f;
#pragma unroll
  for (int t = 0; t < NG; ++t) {
    const int id = threadIdx.x + t * DMA_THREADS;
    if (id < TS::BM * GR) {
      const size_t o = zo + (size_t)(id / GR) * c + (id % GR) * 8;
      ga[t] = *reinterpret_cast<const float4*>(gx + o);
      gb[t] = *reinterpret_cast<const float4*>(gx + o + 4);
      gi[t] = *reinterpret_cast<const uint4*>(g16 + o);
      const uint32_t w[4] = {gi[t].x, gi[t].y, gi[t].z, gi[t].w};
      dot += ga[t].x * __uint_as_float(w[0] << 16) + ga[t].y * __uint_as_float(w[0] & 0xffff0000u) +
             ga[t].z * __uint_as_float(w[1] << 16) + ga[t].w * __uint_as_float(w[1] & 0xffff0000u) +
             gb[t].x * __uint_as_float(w[2] << 16) + gb[t].y * __uint_as_float(w[2] & 0xffff0000u) +
             gb[t].z * __uint_as_float(w[3] << 16) + gb[t].w * __uint_as_float(w[3] & 0xffff0000u);
    }
  }
  return dot;
}

// The partial dots of the Frobenius normalisation's backward as the fused backward kernel forms them (one per tile of
// the fused kernel's tiling, summed in its order), for the unfused launches: the two paths then hand the same bits
// to everything downstream.  Grid (tiles per matrix, matrices); matrices are [r, c] one after the other.
struct NsTileDotParams {
  const float* gx; const uint16_t* g16; float* dot_part;
  int r, c;
};
template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_ns_bwd_dot_tiles(const NsTileDotParams p) {
  __shared__ float red[16];
  constexpr int GR = TS::BN / 8, NG = (TS::BM * GR + DMA_THREADS - 1) / DMA_THREADS;
  const int tc = p.c / TS::BN, member = blockIdx.x, z = blockIdx.y;
  const int rx = member / tc, ry = member % tc;
  const size_t zo = (size_t)z * p.r * p.c + (size_t)rx * TS::BM * p.c + ry * TS::BN;
  float4 ga[NG], gb[NG];
  uint4 gi[NG];
  float dot = ns_tile_dot<TS>(p.gx, p.g16, zo, p.c, ga, gb, gi);
  dot = block_sum(dot, red);
  if (threadIdx.x == 0) p.dot_part[(size_t)z * gridDim.x + member] = dot;
}

// BWD = false: S iterations  A = X X^T;  B = b A + c A A;  X' = a X + B X
// BWD = true:  the same iterations backwards:  Sg = G X^T + X G^T;  H = b Sg + c (Sg A + A Sg);  G' = a G + B G + H X
// TS: 192 x 192 tiles, or 128 x 128 / 128 x 64 when there are too few matrices to fill the chip with the large tile.
template <class TS, bool BWD>
__global__ __launch_bounds__(DMA_THREADS) void k_ns_fused(const NsFusedParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tr = p.r / TS::BM, tc = p.c / TS::BN, ts = p.r / TS::BN;   // tile rows; tile columns of [r, c] and of [r, r]
  const int nbm = tr * tc;                           // blocks per matrix (c >= r: the r x c stages have the most tiles)
  const int L = blockIdx.x, j = L >> 3;
  const int group = (L & 7) + 8 * (j / nbm), member = j % nbm;
  if (group >= p.n) return;
  const int z = p.z0 + group;
  GroupBarrier bar;
  bar.init(p.sync + (size_t)group * 32, nbm, p.error, p.spin_limit, p.sticky);
  const bool sq_tile = member < tr * ts;             // this block owns a tile of the r x r stages
  const int sx = member / ts, sy = member % ts;      // its tile there
  const int rx = member / tc, ry = member % tc;      // its tile of the r x c stages

  if (!BWD && p.g16) {
    // Frobenius normalisation in front of the first iteration: every block of the group sums the same partials
    // in the same order, then scales its own tile of [r, c]
    float ss = 0.f;
    for (int i = 0; i < p.nparts; ++i) ss += p.ss_part[(size_t)(p.part0 + z) * p.nparts + i];
    if (p.part1 >= 0)
      for (int i = 0; i < p.nparts; ++i) ss += p.ss_part[(size_t)(p.part1 + z) * p.nparts + i];
    float n = sqrtf(ss);
    if (p.plain) n = round_bf16(n);
    if (member == 0 && threadIdx.x == 0) p.norms[z] = n;
    float den = n + 1e-7f;
    if (p.plain) den = round_bf16(den);
    const size_t zo = (size_t)z * p.r * p.c + (size_t)rx * TS::BM * p.c + ry * TS::BN;
    constexpr int GR = TS::BN / 8;   // 16-byte granules per tile row
    for (int id = threadIdx.x; id < TS::BM * GR; id += DMA_THREADS) {
      const size_t o = zo + (size_t)(id / GR) * p.c + (id % GR) * 8;
      const uint4 u = *reinterpret_cast<const uint4*>(p.g16 + o);
      const uint32_t w[4] = {u.x, u.y, u.z, u.w};
      float v[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = __fdiv_rn(__uint_as_float(w[i] << 16), den);            // the quotient itself (ttt_operation.py:49), not a product with 1 / den
        v[2 * i + 1] = __fdiv_rn(__uint_as_float(w[i] & 0xffff0000u), den);
      }
      if (p.plain) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = round_bf16(v[i]);
      }
      *reinterpret_cast<float4*>(p.xf[0] + o) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(p.xf[0] + o + 4) = make_float4(v[4], v[5], v[6], v[7]);
      Elem<uint16_t>::store4(p.xb + o, v[0], v[1], v[2], v[3]);
      Elem<uint16_t>::store4(p.xb + o + 4, v[4], v[5], v[6], v[7]);
    }
    bar.sync(p.error);
  }
  LACT_NS_TS(0);
  for (int step = 0; step < p.S; ++step) {
    const int it = BWD ? p.S - 1 - step : step;
    // r and c are made opaque once per iteration: otherwise the compiler hoists every stage's loop-invariant
    // per-lane address registers out of this loop, keeps them all live and spills
    int r = p.r, c = p.c;
    asm volatile("" : "+s"(r), "+s"(c));
    const long long xe = (long long)r * c, se = (long long)r * r;
    const float ca = p.coeffs[3 * it], cb = p.coeffs[3 * it + 1], cc = p.coeffs[3 * it + 2];
    const uint16_t* X = p.xb + it * p.xb_it_stride;
    uint16_t* A = p.ab + it * p.sq_it_stride;
    uint16_t* B = p.bb + it * p.sq_it_stride;
    if (!BWD) {
      const bool last = it + 1 == p.S;
      if (sq_tile) {
        auto q = ns_row_params<1>();
        ns_term(q.g.t[0], X, c, xe, X, c, xe, c);
        q.g.M = r; q.g.N = r; q.g.out = A; q.g.ldo = r; q.g.bso = se;
        q.g.out2 = p.cab; q.g.alpha2 = cc;
        row_gemm_tile<TS, 1, EPI_STORE, false, true>(q, sx, sy, z, smem);
      }
      LACT_NS_TS(1 + step * 6 + 0);
      bar.sync(p.error);
      LACT_NS_TS(1 + step * 6 + 1);
      if (sq_tile) {
        auto q = ns_row_params<1>();
        ns_term(q.g.t[0], p.cab, r, se, A, r, se, r);
        q.g.M = r; q.g.N = r; q.g.out = B; q.g.ldo = r; q.g.bso = se;
        q.g.aux = A; q.g.ldaux = r; q.g.bsaux = se; q.g.alpha = 1.f; q.g.beta = cb;
        row_gemm_tile<TS, 1, EPI_AXPBY, false, true>(q, sx, sy, z, smem);
      }
      LACT_NS_TS(1 + step * 6 + 2);
      bar.sync(p.error);
      LACT_NS_TS(1 + step * 6 + 3);
      {
        auto q = ns_row_params<1>();
        ns_term(q.g.t[0], B, r, se, X, c, xe, r);
        q.g.M = r; q.g.N = c; q.g.ldo = c; q.g.bso = xe;
        q.g.aux = p.xf[it & 1]; q.g.ldaux = c; q.g.bsaux = xe; q.g.alpha = 1.f; q.g.beta = ca;
        q.g.round_out_bf16 = p.plain;
        q.g.out = last ? nullptr : p.xf[(it + 1) & 1];
        q.g.out_c = last ? nullptr : p.xb + (it + 1) * p.xb_it_stride;   // nothing multiplies by the last iterate
        q.g.out_t = last ? p.u_out : nullptr;
        q.g.transpose_mask = p.mask; q.g.nb = p.nb;
        row_gemm_tile<TS, 1, EPI_AXPBY_F32_DUAL, true, true>(q, rx, ry, z, smem);
      }
      LACT_NS_TS(1 + step * 6 + 4);
      bar.sync(p.error);
      LACT_NS_TS(1 + step * 6 + 5);
    } else {
      const int cur = step & 1;
      const uint16_t* gb = p.gxb[cur];
      if (sq_tile) {   // Sg = G X^T + X G^T
        auto q = ns_row_params<2>();
        ns_term(q.g.t[0], gb, c, xe, X, c, xe, c);
        ns_term(q.g.t[1], X, c, xe, gb, c, xe, c);
        q.g.M = r; q.g.N = r; q.g.out = p.sg; q.g.ldo = r; q.g.bso = se;
        row_gemm_tile<TS, 2, EPI_STORE, false, true>(q, sx, sy, z, smem);
      }
      LACT_NS_TS(1 + step * 6 + 0);
      bar.sync(p.error);
      LACT_NS_TS(1 + step * 6 + 1);
      if (sq_tile) {   // H = b Sg + c (Sg A + A Sg)
        auto q = ns_row_params<2>();
        ns_term(q.g.t[0], p.sg, r, se, A, r, se, r);
        ns_term(q.g.t[1], A, r, se, p.sg, r, se, r);
        q.g.M = r; q.g.N = r; q.g.out = p.gas; q.g.ldo = r; q.g.bso = se;
        q.g.aux = p.sg; q.g.ldaux = r; q.g.bsaux = se; q.g.alpha = cc; q.g.beta = cb;
        row_gemm_tile<TS, 2, EPI_AXPBY, false, true>(q, sx, sy, z, smem);
      }
      LACT_NS_TS(1 + step * 6 + 2);
      bar.sync(p.error);
      LACT_NS_TS(1 + step * 6 + 3);
      {                // G' = a G + B G + H X
        auto q = ns_row_params<2>();
        ns_term(q.g.t[0], B, r, se, gb, c, xe, r);
        ns_term(q.g.t[1], p.gas, r, se, X, c, xe, r);
        q.g.M = r; q.g.N = c; q.g.ldo = c; q.g.bso = xe;
        q.g.aux = p.gxf[cur]; q.g.ldaux = c; q.g.bsaux = xe; q.g.alpha = 1.f; q.g.beta = ca;
        q.g.out = p.gxf[cur ^ 1];
        q.g.out_c = step + 1 == p.S ? nullptr : p.gxb[cur ^ 1];   // nothing multiplies by the final gradient
        row_gemm_tile<TS, 2, EPI_AXPBY_F32_DUAL, true, true>(q, rx, ry, z, smem);
      }
      LACT_NS_TS(1 + step * 6 + 4);
      bar.sync(p.error);
      LACT_NS_TS(1 + step * 6 + 5);
    }
  }
  if (BWD && p.dot_part) {
    // the tile this block wrote in the last stage, and the same tile of the bf16 input: 12 granules of 8 elements
    // per thread at 192 x 192, kept in registers for the second pass
    constexpr int GR = TS::BN / 8, NG = (TS::BM * GR + DMA_THREADS - 1) / DMA_THREADS;
    const float* gx = p.gxf[p.S & 1];
    const size_t zo = (size_t)z * p.r * p.c + (size_t)rx * TS::BM * p.c + ry * TS::BN;
    float4 ga[NG], gb[NG];
    uint4 gi[NG];
    // No fence: this tile of gx was written by this very block in the last stage (and in every second stage before),
    // and the waves of a compute unit share its vector L1, which their own stores keep current.  The same holds for
    // every auxiliary tile the blending epilogues read (always the block's own tile of a buffer it wrote itself).
    float dot = ns_tile_dot<TS>(gx, p.g16, zo, p.c, ga, gb, gi);
    dot = block_sum(dot, reinterpret_cast<float*>(smem));
    if (threadIdx.x == 0) p.dot_part[(size_t)z * nbm + member] = dot;
    if (p.gc) {
      bar.sync(p.error);
      float total = 0.f;
      for (int i = 0; i < nbm; ++i) total += __hip_atomic_load(p.dot_part + (size_t)z * nbm + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const float n = p.norms[z];
      float c0 = 1.f / (n + 1e-7f);
      const float c1 = n > 0.f ? total / (n * (n + 1e-7f) * (n + 1e-7f)) : 0.f;
      if (__hip_atomic_load(p.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) c0 = __uint_as_float(0x7fc00000u);
      const float mb = p.mbar ? p.mbar[z % p.nb] : 0.f;
      float md = 0.f;
#pragma unroll
      for (int t = 0; t < NG; ++t) {
        const int id = threadIdx.x + t * DMA_THREADS;
        if (id < TS::BM * GR) {
          const size_t o = zo + (size_t)(id / GR) * p.c + (id % GR) * 8;
          const uint32_t w[4] = {gi[t].x, gi[t].y, gi[t].z, gi[t].w};
          // the gradient that leaves Newton-Schulz through its input cast (G.bfloat16()) has that type
          const float gi0 = __uint_as_float(w[0] << 16), gi1 = __uint_as_float(w[0] & 0xffff0000u), gi2 = __uint_as_float(w[1] << 16),
                      gi3 = __uint_as_float(w[1] & 0xffff0000u), gi4 = __uint_as_float(w[2] << 16), gi5 = __uint_as_float(w[2] & 0xffff0000u),
                      gi6 = __uint_as_float(w[3] << 16), gi7 = __uint_as_float(w[3] & 0xffff0000u);
          float4 v0 = make_float4(ns_input_grad<uint16_t>(ga[t].x, gi0, c0, c1), ns_input_grad<uint16_t>(ga[t].y, gi1, c0, c1),
                                  ns_input_grad<uint16_t>(ga[t].z, gi2, c0, c1), ns_input_grad<uint16_t>(ga[t].w, gi3, c0, c1));
          float4 v1 = make_float4(ns_input_grad<uint16_t>(gb[t].x, gi4, c0, c1), ns_input_grad<uint16_t>(gb[t].y, gi5, c0, c1),
                                  ns_input_grad<uint16_t>(gb[t].z, gi6, c0, c1), ns_input_grad<uint16_t>(gb[t].w, gi7, c0, c1));
          if (p.gm_carry) {
            if (p.carry_valid) {
              const float4 a = *reinterpret_cast<const float4*>(p.gm_carry + o), b = *reinterpret_cast<const float4*>(p.gm_carry + o + 4);
              v0.x += a.x; v0.y += a.y; v0.z += a.z; v0.w += a.w;
              v1.x += b.x; v1.y += b.y; v1.z += b.z; v1.w += b.w;
            }
            if (p.carry_write) {
              *reinterpret_cast<float4*>(p.gm_carry + o) = make_float4(v0.x * mb, v0.y * mb, v0.z * mb, v0.w * mb);
              *reinterpret_cast<float4*>(p.gm_carry + o + 4) = make_float4(v1.x * mb, v1.y * mb, v1.z * mb, v1.w * mb);
            }
            if (p.m_prev) {
              const float4 a = *reinterpret_cast<const float4*>(p.m_prev + o), b = *reinterpret_cast<const float4*>(p.m_prev + o + 4);
              md += v0.x * a.x + v0.y * a.y + v0.z * a.z + v0.w * a.w + v1.x * b.x + v1.y * b.y + v1.z * b.z + v1.w * b.w;
            }
          }
          Elem<uint16_t>::store4(p.gc + o, v0.x, v0.y, v0.z, v0.w);
          Elem<uint16_t>::store4(p.gc + o + 4, v1.x, v1.y, v1.z, v1.w);
        }
      }
      if (p.gm_carry && p.m_prev) {
        __syncthreads();   // the block sum above may still be read from the same LDS words
        md = block_sum(md, reinterpret_cast<float*>(smem));
        if (threadIdx.x == 0) p.mdot_part[(size_t)z * nbm + member] = md;
      }
    }
  }
}

}  // namespace lact
