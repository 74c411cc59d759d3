// bf16 kernels of the TTT operation on the asynchronous-copy main loop (gemm_dma.h).
// Same contractions and epilogues as gemm_kernels.h; all B operands K-contiguous (the host passes the
// transposed bf16 copies of the small matrices where the contraction runs over their leading dimension).
#pragma once
#include "gemm_dma.h"
#include "gemm_kernels.h"

namespace lact {

using TS_ROW = TileShape<256, 128, 2, 2>;   // token-row GEMMs, one accumulator: 128x64 per wave
using TS_SQ = TileShape<128, 128, 2, 2>;    // small square GEMMs (Newton-Schulz) and 2-3 accumulator kernels
using TS_BWD = TileShape<128, 64, 2, 2>;    // six accumulators (update backward): 64x32 per wave
using TS_NS = TileShape<192, 192, 2, 2>;    // 384-multiple square GEMMs (Newton-Schulz at d = dh = 384): 96x96 per wave
using TS_N96 = TileShape<128, 96, 4, 1>;    // Newton-Schulz of few 384-multiple matrices: 12 instead of 9 blocks per 384 x 384 matrix

template <class TS> constexpr int row_stages() { return TS::BM == 128 ? 4 : 3; }

// ------------------------------------------------------------------------------------------------
// k_row_gemm_dma: out[M,N] = epilogue(sum_t A_t[M,K_t] * B_t[N,K_t]^T)
// Extra outputs of the DUAL epilogue: out_ct = transposed copy in bf16 ([N][M] per matrix).
// ------------------------------------------------------------------------------------------------
template <int NT>
struct RowGemmDmaParams {
  RowGemmParams<NT> g;
  uint16_t* out_ct;   // DUAL: bf16 transposed copy [N][M] (batch stride = bso), or null
  TileMap map;        // tiles of M, tiles of N, batch
};

// The phases of one output tile (rows from m0, columns from n0) of batch entry z: one per term.
// B_KS: the B operands are [K, N] (N contiguous) instead of [N, K].
template <class TS, int NT, bool B_KS>
__device__ __forceinline__ void row_gemm_phases(const RowGemmParams<NT>& p, int m0, int n0, int z, DmaPhase<1> (&ph)[NT]) {
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    ph[t].a.base = reinterpret_cast<const uint16_t*>(p.t[t].A) + z * p.t[t].bsA + (size_t)m0 * p.t[t].lda;
    ph[t].a.ld = p.t[t].lda; ph[t].a.rows = p.M - m0; ph[t].a.ks = 0;
    ph[t].b[0].base = reinterpret_cast<const uint16_t*>(p.t[t].B) + z * p.t[t].bsB + (B_KS ? (size_t)n0 : (size_t)n0 * p.t[t].ldb);
    ph[t].b[0].ld = p.t[t].ldb; ph[t].b[0].rows = p.N - n0; ph[t].b[0].ks = B_KS;
    ph[t].nb = 1;
    ph[t].K = p.t[t].K;
  }
}

// EPI_STORE / EPI_AXPBY: the tile staged in LDS as bf16 (StageTile<TS, 2>, = round(acc)) goes out in whole rows; all
// threads of the block take part.
template <class TS, int NT, int EPI>
__device__ __forceinline__ void row_gemm_copy_out_b16(const RowGemmParams<NT>& p, int m0, int n0, int z, const char* smem) {
  using ST = StageTile<TS, 2>;
  const int r0 = ST::row0(), c0 = ST::col0();
  if (ST::active() && n0 + c0 < p.N) {
    const char* src = smem + (r0 * ST::LD + c0) * 2;
    uint16_t* dst = reinterpret_cast<uint16_t*>(p.out) + z * p.bso + (size_t)(m0 + r0) * p.ldo + n0 + c0;
    const uint16_t* aux = reinterpret_cast<const uint16_t*>(p.aux) + z * p.bsaux + (size_t)(m0 + r0) * p.ldaux + n0 + c0;
    const size_t dstep = (size_t)ST::RPP * p.ldo, astep = (size_t)ST::RPP * p.ldaux;
    const bool blend = EPI == EPI_AXPBY || p.accumulate;
    // all auxiliary loads first (no store in between may alias them), then blend and store
    uint4 w[ST::PASSES];
    if (blend) {
      const uint16_t* ap = EPI == EPI_STORE ? dst : aux;
      const size_t st = EPI == EPI_STORE ? dstep : astep;
#pragma unroll
      for (int ps = 0; ps < ST::PASSES; ++ps) {
        const int r = r0 + ps * ST::RPP;
        w[ps] = (r < TS::BM && m0 + r < p.M) ? *reinterpret_cast<const uint4*>(ap + ps * st) : make_uint4(0, 0, 0, 0);
      }
    }
    const float al = EPI == EPI_STORE ? 1.f : p.alpha, be = EPI == EPI_STORE ? 1.f : p.beta;
    uint16_t* dst2 = (EPI == EPI_STORE && p.out2) ? reinterpret_cast<uint16_t*>(p.out2) + (dst - reinterpret_cast<uint16_t*>(p.out)) : nullptr;
    // LDS reads in unconditional groups of 8 (a branch per row would put every read's latency in line)
    uint4 ug[8];
#pragma unroll
    for (int ps = 0; ps < ST::PASSES; ++ps) {
      if (ps % 8 == 0) {
#pragma unroll
        for (int g = 0; g < 8; ++g)
          if (ps + g < ST::PASSES) ug[g] = ST::read16(src, r0, ps + g);
      }
      const int r = r0 + ps * ST::RPP;
      if (r < TS::BM && m0 + r < p.M) {
        uint4 u = ug[ps % 8];
        if (blend) {
          // the staged values are round(acc); each product and the sum are tensors of their own in the reference
          uint32_t uu[4] = {u.x, u.y, u.z, u.w}, ww[4] = {w[ps].x, w[ps].y, w[ps].z, w[ps].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float lo = round_bf16(al * __uint_as_float(uu[j] << 16)) + round_bf16(be * __uint_as_float(ww[j] << 16));
            const float hi = round_bf16(al * __uint_as_float(uu[j] & 0xffff0000u)) + round_bf16(be * __uint_as_float(ww[j] & 0xffff0000u));
            uu[j] = (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
          }
          u = make_uint4(uu[0], uu[1], uu[2], uu[3]);
        }
        *reinterpret_cast<uint4*>(dst) = u;
        if (dst2) {
          uint32_t uu[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
          for (int j = 0; j < 4; ++j)
            uu[j] = (uint32_t)f32_to_bf16(p.alpha2 * __uint_as_float(uu[j] << 16)) |
                    ((uint32_t)f32_to_bf16(p.alpha2 * __uint_as_float(uu[j] & 0xffff0000u)) << 16);
          *reinterpret_cast<uint4*>(dst2) = make_uint4(uu[0], uu[1], uu[2], uu[3]);
        }
      }
      dst += dstep;
      if (dst2) dst2 += dstep;
    }
  }
}

// Transposed copies of the fp32 tile staged in LDS (StageTile<TS, 4>): lanes run along n (conflict-free LDS reads),
// each lane owns 8 consecutive m.  All threads of the block take part.
template <class TS, int NT>
__device__ __forceinline__ void row_gemm_copy_out_transposed(const RowGemmParams<NT>& p, uint16_t* out_ct, bool tr, int m0, int n0, int z, const char* smem) {
  using ST = StageTile<TS, 4>;
  const float* tile = reinterpret_cast<const float*>(smem);
#pragma unroll 2
  for (int id = threadIdx.x; id < TS::BN * (TS::BM / 8); id += DMA_THREADS) {
    const int nl = id % TS::BN, ml = (id / TS::BN) * 8;
    const int m = m0 + ml, n = n0 + nl;
    if (m >= p.M || n >= p.N) continue;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = tile[(ml + j) * ST::LD + nl];
    const size_t off = z * p.bso + (size_t)n * p.M + m;
    if (p.out_t && tr) {
      Elem<float>::store4(p.out_t + off, v[0], v[1], v[2], v[3]);
      Elem<float>::store4(p.out_t + off + 4, v[4], v[5], v[6], v[7]);
    }
    if (out_ct) {
      Elem<uint16_t>::store4(out_ct + off, v[0], v[1], v[2], v[3]);
      Elem<uint16_t>::store4(out_ct + off + 4, v[4], v[5], v[6], v[7]);
    }
  }
}

// One output tile (bx, by) of batch entry z.  B_KS: the B operands are [K, N] (N contiguous) instead of [N, K].
// SC1: the operands were written by other compute units during this kernel (loads bypass the vector L1); the
// auxiliary tile of the blending epilogues is always one this block wrote itself or an earlier kernel wrote.
// All threads of the block must call it; on return the LDS may still be read by this block's epilogue, so the
// caller synchronises the block before the LDS is written again.
template <class TS, int NT, int EPI, bool B_KS, bool SC1>
__device__ __forceinline__ void row_gemm_tile(const RowGemmDmaParams<NT>& pp, int bx, int by, int z, char* smem) {
  constexpr int STAGES = row_stages<TS>();
  using Pipe = DmaPipe<TS, 1, NT, STAGES, SC1>;
  const RowGemmParams<NT>& p = pp.g;
  const int m0 = bx * TS::BM, n0 = by * TS::BN;
  DmaPhase<1> ph[NT];
  row_gemm_phases<TS, NT, B_KS>(p, m0, n0, z, ph);
  f32x16 acc[1][TS::TM][TS::TN];   // defined on the matrix waves' path only: the loader waves' registers stay free for their copies
  LACT_TS(0);
  Pipe pipe(smem, ph);
  const bool loader = Pipe::is_loader();
  LACT_TS(1);
  if (loader) {
    pipe.template load_all<Pipe::loads(1)>();
  } else {
    zero_acc<TS>(acc[0]);
    int step = 0;
#pragma unroll
    for (int t = 0; t < NT; ++t) pipe.template run_phase<1, false, B_KS>(p.t[t].K / DMA_BK, step, acc);
  }
  __syncthreads();
  LACT_TS(2);

  // ---- epilogue through an LDS-staged tile (see StageTile)
  if (EPI != EPI_AXPBY_F32_DUAL) {
    using ST = StageTile<TS, 2>;
    char* lb = smem + ST::lane_base();
    if (!loader) {
      LACT_FOR_QUADS(TS) ST::put4(lb, tm, tn, g, acc[0][tm][tn][4 * g], acc[0][tm][tn][4 * g + 1], acc[0][tm][tn][4 * g + 2], acc[0][tm][tn][4 * g + 3]);
    }
    __syncthreads();
    row_gemm_copy_out_b16<TS, NT, EPI>(p, m0, n0, z, smem);
  } else {
    using ST = StageTile<TS, 4>;
    char* lb = smem + ST::lane_base();
    if (!loader) {
      LACT_FOR_QUADS(TS) ST::put4(lb, tm, tn, g, acc[0][tm][tn][4 * g], acc[0][tm][tn][4 * g + 1], acc[0][tm][tn][4 * g + 2], acc[0][tm][tn][4 * g + 3]);
    }
    __syncthreads();
    const bool tr = (p.transpose_mask >> (z / p.nb)) & 1;
    const bool need_t = (p.out_t && tr) || pp.out_ct;
    const int r0 = ST::row0(), c0 = ST::col0();
    if (ST::active() && n0 + c0 < p.N) {
      char* src = smem + (r0 * ST::LD + c0) * 4;
      size_t off = z * p.bso + (size_t)(m0 + r0) * p.ldo + n0 + c0;
      const float* aux = reinterpret_cast<const float*>(p.aux) + z * p.bsaux + (size_t)(m0 + r0) * p.ldaux + n0 + c0;
      const size_t dstep = (size_t)ST::RPP * p.ldo, astep = (size_t)ST::RPP * p.ldaux;
      float4 x4[ST::PASSES];
#pragma unroll
      for (int ps = 0; ps < ST::PASSES; ++ps) {
        const int r = r0 + ps * ST::RPP;
        x4[ps] = (r < TS::BM && m0 + r < p.M) ? *reinterpret_cast<const float4*>(aux + ps * astep) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
      uint4 ag[8];
#pragma unroll
      for (int ps = 0; ps < ST::PASSES; ++ps) {
        if (ps % 8 == 0) {
#pragma unroll
          for (int g = 0; g < 8; ++g)
            if (ps + g < ST::PASSES) ag[g] = ST::read16(src, r0, ps + g);
        }
        const int r = r0 + ps * ST::RPP;
        if (r < TS::BM && m0 + r < p.M) {
          float4* sp = reinterpret_cast<float4*>(src + ps * ST::RPP * ST::LD * 4);
          const float4 a4 = __builtin_bit_cast(float4, ag[ps % 8]);
          // the matrix product is a bf16 tensor in the reference (ttt_operation.py:62)
          float v[4] = {dual_blend(__fmul_rn(p.alpha, round_bf16(a4.x)), __fmul_rn(p.beta, x4[ps].x), p.round_out_bf16),
                        dual_blend(__fmul_rn(p.alpha, round_bf16(a4.y)), __fmul_rn(p.beta, x4[ps].y), p.round_out_bf16),
                        dual_blend(__fmul_rn(p.alpha, round_bf16(a4.z)), __fmul_rn(p.beta, x4[ps].z), p.round_out_bf16),
                        dual_blend(__fmul_rn(p.alpha, round_bf16(a4.w)), __fmul_rn(p.beta, x4[ps].w), p.round_out_bf16)};
          if (p.out) Elem<float>::store4(reinterpret_cast<float*>(p.out) + off, v[0], v[1], v[2], v[3]);
          if (p.out_c) Elem<uint16_t>::store4(reinterpret_cast<uint16_t*>(p.out_c) + off, v[0], v[1], v[2], v[3]);
          if (p.out_t && !tr) Elem<float>::store4(p.out_t + off, v[0], v[1], v[2], v[3]);
          if (need_t) *sp = make_float4(v[0], v[1], v[2], v[3]);
        }
        off += dstep;
      }
    }
    if (need_t) {
      __syncthreads();
      row_gemm_copy_out_transposed<TS, NT>(p, pp.out_ct, tr, m0, n0, z, smem);
    }
  }
  LACT_TS(3);
}

template <class TS, int NT, int EPI, bool B_KS>
__global__ __launch_bounds__(DMA_THREADS) void k_row_gemm_dma(const RowGemmDmaParams<NT> pp) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int bx, by, z;
  if (!pp.map.locate(blockIdx.x, bx, by, z)) return;
  row_gemm_tile<TS, NT, EPI, B_KS, false>(pp, bx, by, z, smem);
}

// ------------------------------------------------------------------------------------------------
// Hidden-layer kernels.  W1T / G1T: transposed copies ([dh, d]) of w1 and of its gradient-of-gradient.
// ------------------------------------------------------------------------------------------------
struct HiddenDmaParams {
  HiddenParams h;
  TileMap map;   // token tiles, hidden tiles, batch
};

template <class TS>
__device__ __forceinline__ DmaOperand token_operand(const void* base, long long bs, int ld, int z, int m0, int T) {
  DmaOperand o;
  o.base = reinterpret_cast<const uint16_t*>(base) + z * bs + (size_t)m0 * ld;
  o.ld = ld;
  o.rows = T - m0;
  o.ks = 0;
  return o;
}
__device__ __forceinline__ DmaOperand weight_operand(const void* base, long long bs, int ld, int z, int n0, int rows) {
  DmaOperand o;
  o.base = reinterpret_cast<const uint16_t*>(base) + z * bs + (size_t)n0 * ld;
  o.ld = ld;
  o.rows = rows - n0;
  o.ks = 0;
  return o;
}
// [K, rows] matrix (rows contiguous): the tile starts at column n0
__device__ __forceinline__ DmaOperand weight_operand_ks(const void* base, long long bs, int ld, int z, int n0, int rows) {
  DmaOperand o;
  o.base = reinterpret_cast<const uint16_t*>(base) + z * bs + n0;
  o.ld = ld;
  o.rows = rows - n0;
  o.ks = 1;
  return o;
}

// apply forward: O0 = silu(X W0^T) * (X W2^T)
template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_apply_hidden_dma(const HiddenDmaParams pp) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int STAGES = 3;
  using Pipe = DmaPipe<TS, 2, 1, STAGES>;
  const HiddenParams& p = pp.h;
  int bx, by, z;
  if (!pp.map.locate(blockIdx.x, bx, by, z)) return;
  const int m0 = bx * TS::BM, n0 = by * TS::BN;
  DmaPhase<2> ph[1];
  ph[0].a = token_operand<TS>(p.X, p.bsx, p.ldx, z, m0, p.T);
  ph[0].b[0] = weight_operand(p.W0, p.bsw, p.d, z, n0, p.dh);
  ph[0].b[1] = weight_operand(p.W2, p.bsw, p.d, z, n0, p.dh);
  ph[0].nb = 2;
  ph[0].K = p.d;
  const int nk = (p.d + DMA_BK - 1) / DMA_BK;
  f32x16 acc[2][TS::TM][TS::TN];
  LACT_TS(0);
  Pipe pipe(smem, ph);
  const bool loader = Pipe::is_loader();
  LACT_TS(1);
  if (loader) {
    pipe.template load_all<Pipe::loads(2)>();
  } else {
    zero_acc<TS>(acc[0]);
    zero_acc<TS>(acc[1]);
    int step = 0;
    pipe.template run_phase<2>(nk, step, acc);
  }
  __syncthreads();
  LACT_TS(2);
  using SB = StageTile<TS, 2>;
  if (!loader) {
    LACT_FOR_QUADS(TS) {
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float y0 = round_bf16(acc[0][tm][tn][4 * g + j]), y2 = round_bf16(acc[1][tm][tn][4 * g + j]);
        v[j] = round_bf16(y0 * sigmoidf_(y0)) * y2;
      }
      SB::put4(smem + SB::lane_base(), tm, tn, g, v[0], v[1], v[2], v[3]);
    }
  }
  __syncthreads();
  LACT_TS(3);
  copy_out_b16<TS>(smem, reinterpret_cast<uint16_t*>(p.O0) + z * p.bso + (size_t)m0 * p.dh + n0, p.dh, p.T - m0, p.dh - n0);
  LACT_TS(4);
}

// Shared main loop of the three-accumulator kernels: acc0 = X W0^T, acc1 = X W2^T, acc2 = Y W1 (via W1T).
template <class TS>
__device__ __forceinline__ void three_acc_mainloop(const HiddenDmaParams& pp, char* smem, int m0, int n0, int z,
                                                   f32x16 (&a02)[2][TS::TM][TS::TN], f32x16 (&a1)[1][TS::TM][TS::TN]) {
  constexpr int STAGES = 3;
  using Pipe = DmaPipe<TS, 2, 2, STAGES>;
  const HiddenParams& p = pp.h;
  DmaPhase<2> ph[2];
  ph[0].a = token_operand<TS>(p.X, p.bsx, p.ldx, z, m0, p.T);
  ph[0].b[0] = weight_operand(p.W0, p.bsw, p.d, z, n0, p.dh);
  ph[0].b[1] = weight_operand(p.W2, p.bsw, p.d, z, n0, p.dh);
  ph[0].nb = 2;
  ph[0].K = p.d;
  ph[1].a = token_operand<TS>(p.Y, p.bsy, p.ldy, z, m0, p.T);
  ph[1].b[0] = weight_operand_ks(p.W1, p.bsw, p.dh, z, n0, p.dh);   // V * W1: w1 is [d, dh]
  ph[1].b[1] = ph[1].b[0];
  ph[1].nb = 1;
  ph[1].K = p.d;
  const int nk = (p.d + DMA_BK - 1) / DMA_BK;
  Pipe pipe(smem, ph);
  if (Pipe::is_loader()) {
    pipe.template load_all<Pipe::loads(1)>();
  } else {
    zero_acc<TS>(a02[0]);
    zero_acc<TS>(a02[1]);
    zero_acc<TS>(a1[0]);
    int step = 0;
    pipe.template run_phase<2>(nk, step, a02);
    pipe.template run_phase<1, false, true>(nk, step, a1);
  }
  __syncthreads();
}

// bf16 pairs of a 16-byte granule <-> eight floats
__device__ __forceinline__ void unpack8(const uint4& u, float (&f)[8]) {
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_bf16(f[2 * i]) | ((uint32_t)f32_to_bf16(f[2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// update forward.  O0 = dgate_before_act, O1 = hidden * lr1, O2 = dhidden_before_mul (the operands of the three
// fast-weight gradient GEMMs: lr0 and lr2 scale k there, ttt_operation.py:166-168).  For the backward, when O3 is set:
// O3..O5 = the rounded pre-activations, O6 = O0 * lr0, O7 = O2 * lr2.
// Epilogue: the matrix waves stage only the three rounded products; the pointwise chain (the vector-ALU bulk of this
// kernel) then runs on all eight waves, row-wise -- a thread owns eight consecutive columns of four rows -- and every
// output goes from registers straight to whole 16-byte row segments: half the vector-ALU time per thread and three
// staged tiles instead of eight.  Element by element the same operations on the same rounded values as before.
// The three accumulators of a hidden-stage tile, rounded to bf16, into three staged tiles at the start of the ring
// (matrix waves only; the caller synchronises the block before anyone reads them).
template <class TS>
__device__ __forceinline__ void stage_three_products(char* smem, const f32x16 (&a02)[2][TS::TM][TS::TN], const f32x16 (&a1)[1][TS::TM][TS::TN]) {
  using SB = StageTile<TS, 2>;
  static_assert(3 * SB::BYTES <= DmaSmem<TS, 2, 3>::BYTES, "the three staged tiles lie in the ring");
  char* s0 = smem + SB::lane_base(); char* s1 = s0 + SB::BYTES; char* s2 = s0 + 2 * SB::BYTES;
  if (threadIdx.x < TS::THREADS) LACT_FOR_QUADS(TS) {
    SB::put4(s0, tm, tn, g, a02[0][tm][tn][4 * g], a02[0][tm][tn][4 * g + 1], a02[0][tm][tn][4 * g + 2], a02[0][tm][tn][4 * g + 3]);
    SB::put4(s1, tm, tn, g, a02[1][tm][tn][4 * g], a02[1][tm][tn][4 * g + 1], a02[1][tm][tn][4 * g + 2], a02[1][tm][tn][4 * g + 3]);
    SB::put4(s2, tm, tn, g, a1[0][tm][tn][4 * g], a1[0][tm][tn][4 * g + 1], a1[0][tm][tn][4 * g + 2], a1[0][tm][tn][4 * g + 3]);
  }
}

template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_update_hidden_dma(const HiddenDmaParams pp) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const HiddenParams& p = pp.h;
  int bx, by, z;
  if (!pp.map.locate(blockIdx.x, bx, by, z)) return;
  const int m0 = bx * TS::BM, n0 = by * TS::BN;
  using SB = StageTile<TS, 2>;
  {
    f32x16 a02[2][TS::TM][TS::TN], a1[1][TS::TM][TS::TN];
    three_acc_mainloop<TS>(pp, smem, m0, n0, z, a02, a1);
    stage_three_products<TS>(smem, a02, a1);
  }
  __syncthreads();
  if (!SB::active()) return;
  const int r0 = SB::row0(), c0 = SB::col0();
  if (n0 + c0 >= p.dh) return;
  const bool keep = p.O3 != nullptr;
  const char* src = smem + (r0 * SB::LD + c0) * 2;
  size_t off = z * p.bso + (size_t)(m0 + r0) * p.dh + n0 + c0;
  const size_t step = (size_t)SB::RPP * p.dh;
  // all LDS reads and the learning rates of this thread's rows first: their latencies overlap
  uint4 ug[SB::PASSES], uh[SB::PASSES], ud[SB::PASSES];
  float l0[SB::PASSES], l1[SB::PASSES], l2[SB::PASSES];
#pragma unroll
  for (int ps = 0; ps < SB::PASSES; ++ps) {
    ug[ps] = SB::read16(src, r0, ps);
    uh[ps] = SB::read16(src + SB::BYTES, r0, ps);
    ud[ps] = SB::read16(src + 2 * SB::BYTES, r0, ps);
    const int m = m0 + r0 + ps * SB::RPP;
    const bool mv = r0 + ps * SB::RPP < TS::BM && m < p.T;
    l0[ps] = mv ? p.lr0[z * p.bslr + m] : 0.f;
    l1[ps] = mv ? p.lr1[z * p.bslr + m] : 0.f;
    l2[ps] = mv ? p.lr2[z * p.bslr + m] : 0.f;
  }
#pragma unroll
  for (int ps = 0; ps < SB::PASSES; ++ps) {
    const int r = r0 + ps * SB::RPP;
    if (r < TS::BM && m0 + r < p.T) {
      float gg[8], h2[8], dh[8], z0[8], z1[8], z2[8], y0[8], y2[8];
      unpack8(ug[ps], gg);
      unpack8(uh[ps], h2);
      unpack8(ud[ps], dh);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const UpdatePointwise u = update_pointwise<uint16_t>(gg[j], h2[j], dh[j], silu_parts(gg[j]));
        z0[j] = u.dgpre; z1[j] = u.hid * l1[ps]; z2[j] = u.dh2;
        y0[j] = u.dgpre * l0[ps]; y2[j] = u.dh2 * l2[ps];
      }
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O0) + off) = pack8(z0);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O1) + off) = pack8(z1);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O2) + off) = pack8(z2);
      if (keep) {   // the backward is going to start from the rounded pre-activations instead of recomputing them
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O3) + off) = ug[ps];
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O4) + off) = uh[ps];
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O5) + off) = ud[ps];
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O6) + off) = pack8(y0);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O7) + off) = pack8(y2);
      }
    }
    off += step;
  }
}

// apply backward, hidden stage: Y0 = X W0^T, Y2 = X W2^T, GH = dOut W1 -> O0 = silu(Y0) * Y2 (the hidden activation,
// recomputed), O1 = d Y0, O2 = d Y2 (lact_swiglu_ffn.py:46-76).  Epilogue as in k_update_hidden_dma: three staged
// products, the pointwise part on all eight waves, stores straight from registers.
template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_apply_bwd_hidden_dma(const HiddenDmaParams pp) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const HiddenParams& p = pp.h;
  int bx, by, z;
  if (!pp.map.locate(blockIdx.x, bx, by, z)) return;
  const int m0 = bx * TS::BM, n0 = by * TS::BN;
  using SB = StageTile<TS, 2>;
  {
    f32x16 a02[2][TS::TM][TS::TN], a1[1][TS::TM][TS::TN];
    three_acc_mainloop<TS>(pp, smem, m0, n0, z, a02, a1);
    stage_three_products<TS>(smem, a02, a1);
  }
  __syncthreads();
  if (!SB::active()) return;
  const int r0 = SB::row0(), c0 = SB::col0();
  if (n0 + c0 >= p.dh) return;
  const char* src = smem + (r0 * SB::LD + c0) * 2;
  size_t off = z * p.bso + (size_t)(m0 + r0) * p.dh + n0 + c0;
  const size_t step = (size_t)SB::RPP * p.dh;
  uint4 u0[SB::PASSES], u2[SB::PASSES], ug[SB::PASSES];
#pragma unroll
  for (int ps = 0; ps < SB::PASSES; ++ps) {
    u0[ps] = SB::read16(src, r0, ps);
    u2[ps] = SB::read16(src + SB::BYTES, r0, ps);
    ug[ps] = SB::read16(src + 2 * SB::BYTES, r0, ps);
  }
#pragma unroll
  for (int ps = 0; ps < SB::PASSES; ++ps) {
    const int r = r0 + ps * SB::RPP;
    if (r < TS::BM && m0 + r < p.T) {
      float y0[8], y2[8], gh[8], hq[8], gy0[8], gy2[8];
      unpack8(u0[ps], y0);
      unpack8(u2[ps], y2);
      unpack8(ug[ps], gh);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const SiluParts sp = silu_parts(y0[j]);
        const float sg = round_bf16(sp.silu);
        hq[j] = sg * y2[j]; gy0[j] = round_bf16(gh[j] * y2[j]) * sp.d1; gy2[j] = gh[j] * sg;
      }
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O0) + off) = pack8(hq);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O1) + off) = pack8(gy0);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O2) + off) = pack8(gy2);
    }
    off += step;
  }
}

// update backward, hidden stage: phases (X; W0,W2), (X; G0,G2), (Y; W1T,G1T)
template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_update_bwd_hidden_dma(const HiddenDmaParams pp) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int STAGES = 3;
  using Pipe = DmaPipe<TS, 2, 3, STAGES>;
  const HiddenParams& p = pp.h;
  int bx, by, z;
  if (!pp.map.locate(blockIdx.x, bx, by, z)) return;
  const int m0 = bx * TS::BM, n0 = by * TS::BN;
  DmaPhase<2> ph[3];
  ph[0].a = token_operand<TS>(p.X, p.bsx, p.ldx, z, m0, p.T);
  ph[0].b[0] = weight_operand(p.W0, p.bsw, p.d, z, n0, p.dh);
  ph[0].b[1] = weight_operand(p.W2, p.bsw, p.d, z, n0, p.dh);
  ph[1].a = ph[0].a;
  ph[1].b[0] = weight_operand(p.G0, p.bsw, p.d, z, n0, p.dh);
  ph[1].b[1] = weight_operand(p.G2, p.bsw, p.d, z, n0, p.dh);
  ph[2].a = token_operand<TS>(p.Y, p.bsy, p.ldy, z, m0, p.T);
  ph[2].b[0] = weight_operand_ks(p.W1, p.bsw, p.dh, z, n0, p.dh);
  ph[2].b[1] = weight_operand_ks(p.G1, p.bsw, p.dh, z, n0, p.dh);
  ph[0].K = ph[1].K = ph[2].K = p.d;
  ph[0].nb = ph[1].nb = ph[2].nb = 2;
  const int nk = (p.d + DMA_BK - 1) / DMA_BK;
  f32x16 aw[2][TS::TM][TS::TN], ag[2][TS::TM][TS::TN], ay[2][TS::TM][TS::TN];
  Pipe pipe(smem, ph);
  const bool loader = Pipe::is_loader();
  if (loader) {
    pipe.template load_all<Pipe::loads(2)>();
  } else {
    zero_acc<TS>(aw[0]); zero_acc<TS>(aw[1]); zero_acc<TS>(ag[0]); zero_acc<TS>(ag[1]); zero_acc<TS>(ay[0]); zero_acc<TS>(ay[1]);
    int step = 0;
    pipe.template run_phase<2>(nk, step, aw);
    pipe.template run_phase<2>(nk, step, ag);
    pipe.template run_phase<2, false, true>(nk, step, ay);
  }
  __syncthreads();
  // Epilogue: the six rounded products staged as bf16 tiles, then the pointwise part on all eight waves, row-wise (a
  // thread owns 8 consecutive columns of two rows), results straight from registers to 16-byte row segments.
  using SB = StageTile<TS, 2>;
  static_assert(TS::BN == 64 && TS::WAVES_N == 2, "a row is 8 granules: four per wave column");
  {
    char* lb = smem + SB::lane_base();
    if (!loader) LACT_FOR_QUADS(TS) {
      SB::put4(lb + 0 * SB::BYTES, tm, tn, g, aw[0][tm][tn][4 * g], aw[0][tm][tn][4 * g + 1], aw[0][tm][tn][4 * g + 2], aw[0][tm][tn][4 * g + 3]);
      SB::put4(lb + 1 * SB::BYTES, tm, tn, g, aw[1][tm][tn][4 * g], aw[1][tm][tn][4 * g + 1], aw[1][tm][tn][4 * g + 2], aw[1][tm][tn][4 * g + 3]);
      SB::put4(lb + 2 * SB::BYTES, tm, tn, g, ay[0][tm][tn][4 * g], ay[0][tm][tn][4 * g + 1], ay[0][tm][tn][4 * g + 2], ay[0][tm][tn][4 * g + 3]);
      SB::put4(lb + 3 * SB::BYTES, tm, tn, g, ag[0][tm][tn][4 * g], ag[0][tm][tn][4 * g + 1], ag[0][tm][tn][4 * g + 2], ag[0][tm][tn][4 * g + 3]);
      SB::put4(lb + 4 * SB::BYTES, tm, tn, g, ay[1][tm][tn][4 * g], ay[1][tm][tn][4 * g + 1], ay[1][tm][tn][4 * g + 2], ay[1][tm][tn][4 * g + 3]);
      SB::put4(lb + 5 * SB::BYTES, tm, tn, g, ag[1][tm][tn][4 * g], ag[1][tm][tn][4 * g + 1], ag[1][tm][tn][4 * g + 2], ag[1][tm][tn][4 * g + 3]);
    }
  }
  __syncthreads();
  const int r0 = SB::row0(), c0 = SB::col0();
  const bool nv = n0 + c0 < p.dh;
  const char* src = smem + (r0 * SB::LD + c0) * 2;
  size_t off = z * p.bso + (size_t)(m0 + r0) * p.dh + n0 + c0;
  const size_t step = (size_t)SB::RPP * p.dh;
  uint4 u[SB::PASSES][6];
  float l0[SB::PASSES], l1[SB::PASSES], l2[SB::PASSES];
#pragma unroll
  for (int ps = 0; ps < SB::PASSES; ++ps) {
#pragma unroll
    for (int i = 0; i < 6; ++i) u[ps][i] = SB::read16(src + i * SB::BYTES, r0, ps);
    const int m = m0 + r0 + ps * SB::RPP;
    const bool mv = r0 + ps * SB::RPP < TS::BM && m < p.T;
    l0[ps] = mv ? p.lr0[z * p.bslr + m] : 0.f;
    l1[ps] = mv ? p.lr1[z * p.bslr + m] : 0.f;
    l2[ps] = mv ? p.lr2[z * p.bslr + m] : 0.f;
  }
#pragma unroll
  for (int ps = 0; ps < SB::PASSES; ++ps) {
    const int r = r0 + ps * SB::RPP, m = m0 + r;
    const bool mv = r < TS::BM && m < p.T;
    float gg[8], h2[8], dh[8], gz0[8], gz1[8], gz2[8], o0[8], o1[8], o2[8], o3[8], o4[8], o5[8];
    unpack8(u[ps][0], gg); unpack8(u[ps][1], h2); unpack8(u[ps][2], dh);
    unpack8(u[ps][3], gz0); unpack8(u[ps][4], gz1); unpack8(u[ps][5], gz2);
    float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const SiluParts sp = silu_parts(gg[j]);
      const UpdatePointwise up = update_pointwise<uint16_t>(gg[j], h2[j], dh[j], sp);
      if (mv && nv) { s0 += gz0[j] * up.dgpre; s1 += gz1[j] * up.hid; s2 += gz2[j] * up.dh2; }
      const float ghid = gz1[j] * l1[ps], gdh2 = gz2[j] * l2[ps], gdg = gz0[j] * l0[ps];
      o0[j] = ghid * h2[j] * sp.d1 + gdh2 * dh[j] * sp.d1 + gdg * dh[j] * h2[j] * sp.d2;
      o1[j] = gdh2 * sp.silu + gdg * h2[j] * sp.d1;
      o2[j] = ghid * sp.silu + gdg * dh[j] * sp.d1;
      o3[j] = up.dgpre * l0[ps]; o4[j] = up.hid * l1[ps]; o5[j] = up.dh2 * l2[ps];
    }
    // learning-rate gradients: one partial per (row, wave column of 32 columns) = four lanes, slots as before
    s0 += __shfl_xor(s0, 1, 64); s1 += __shfl_xor(s1, 1, 64); s2 += __shfl_xor(s2, 1, 64);
    s0 += __shfl_xor(s0, 2, 64); s1 += __shfl_xor(s1, 2, 64); s2 += __shfl_xor(s2, 2, 64);
    if (mv) {
      if (nv) {
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O0) + off) = pack8(o0);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O1) + off) = pack8(o1);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O2) + off) = pack8(o2);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O3) + off) = pack8(o3);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O4) + off) = pack8(o4);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O5) + off) = pack8(o5);
      }
      if ((threadIdx.x & 3) == 0) {
        const size_t lo = (size_t)(by * TS::WAVES_N + ((threadIdx.x & 7) >> 2)) * p.lrpart_stride + (size_t)z * p.Tcap + m;
        p.lrpart[0 * p.lrpart_mat_stride + lo] = s0;
        p.lrpart[1 * p.lrpart_mat_stride + lo] = s1;
        p.lrpart[2 * p.lrpart_mat_stride + lo] = s2;
      }
    }
    off += step;
  }
}

// update backward, hidden stage, from the pre-activations the forward kept (I0 = k W0^T, I1 = k W2^T, I2 = v W1,
// rounded as the forward rounded them): only the three products with the gradient matrices are left,
// phases (X; G0, G2) and (Y; G1 read K-strided).  O0..O2 as in k_update_bwd_hidden_dma; what that kernel writes
// to O3..O5 are the forward's own lr-scaled operands, which the forward kept as well.
// The block's three input tiles travel through the ring like operands: a last phase of one or two K-steps copies
// columns [64h, 64h + 64) of I0, I1, I2 into the A, B0, B1 places of a stage, where they simply stay -- the matrix
// waves only pass the barriers of those K-steps.  Every lane then finds the inputs of its accumulator positions
// in those stages (same swizzle as any operand tile), overwrites them with the results, and the block copies the
// stages out.  dh must be a multiple of 64.
template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_update_bwd_hidden_kept_dma(const HiddenDmaParams pp) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  static_assert(TS::BM == 128 && TS::BN == 128 && TS::WN == 64, "one wave column per 64-column half of the tile");
  constexpr int STAGES = 3;
  using Pipe = DmaPipe<TS, 2, 3, STAGES>;
  using SM = typename Pipe::SM;
  const HiddenParams& p = pp.h;
  int bx, by, z;
  if (!pp.map.locate(blockIdx.x, bx, by, z)) return;
  const int m0 = bx * TS::BM, n0 = by * TS::BN;
  const int nk = p.d / DMA_BK;
  const int halves = min(TS::BN, p.dh - n0) / 64;          // valid 64-column halves of this tile
  DmaPhase<2> ph[3];
  // the one-accumulator phase first: the two-accumulator K-steps in front of the input stages are the longer ones,
  // which gives the input copies more time to land
  ph[0].a = token_operand<TS>(p.Y, p.bsy, p.ldy, z, m0, p.T);
  ph[0].b[0] = weight_operand_ks(p.G1, p.bsw, p.dh, z, n0, p.dh);
  ph[0].b[1] = ph[0].b[0];
  ph[0].nb = 1;
  ph[0].K = p.d;
  ph[1].a = token_operand<TS>(p.X, p.bsx, p.ldx, z, m0, p.T);
  ph[1].b[0] = weight_operand(p.G0, p.bsw, p.d, z, n0, p.dh);
  ph[1].b[1] = weight_operand(p.G2, p.bsw, p.d, z, n0, p.dh);
  ph[1].nb = 2;
  ph[1].K = p.d;
  ph[2].a = token_operand<TS>(reinterpret_cast<const uint16_t*>(p.I0) + n0, p.bsi, p.dh, z, m0, p.T);
  ph[2].b[0] = token_operand<TS>(reinterpret_cast<const uint16_t*>(p.I1) + n0, p.bsi, p.dh, z, m0, p.T);
  ph[2].b[1] = token_operand<TS>(reinterpret_cast<const uint16_t*>(p.I2) + n0, p.bsi, p.dh, z, m0, p.T);
  ph[2].nb = 2;
  ph[2].K = halves * 64;
  f32x16 ag[2][TS::TM][TS::TN], ay[1][TS::TM][TS::TN];
  LACT_TS(0);
  Pipe pipe(smem, ph);
  const bool loader = Pipe::is_loader();
  if (loader) {
    pipe.template load_all<Pipe::loads(1)>();
  } else {
    zero_acc<TS>(ag[0]);
    zero_acc<TS>(ag[1]);
    zero_acc<TS>(ay[0]);
    int step = 0;
    pipe.template run_phase<1, false, true>(nk, step, ay);
    pipe.template run_phase<2>(nk, step, ag);
    LACT_TS(1);
    for (int i = 0; i < halves; ++i) __syncthreads();   // the input stages land behind these barriers
  }
  LACT_TS(2);
  // Input half h sits in the stage of K-step 2 nk + h; the stage of K-step 2 nk + 2 (= the last real K-step's, which
  // every matrix wave has left: it has passed a barrier since its last fetch) is free.  Per half: the two matrix waves
  // that own its 64 columns put their three rounded products there, in the layout of the input stage beside it; then
  // all eight waves run the pointwise part row-wise -- a thread owns one 16-byte granule (8 columns) of two rows --
  // and store the three results straight from registers.  Half the vector-ALU work per thread of a matrix-waves-only
  // epilogue, and no staged result tiles.
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  char* fz = smem + ((2 * nk + 2) % STAGES) * SM::STAGE;
  const size_t off = z * p.bso + (size_t)m0 * p.dh + n0;
  for (int h = 0; h < halves; ++h) {
    if (!loader && wave % TS::WAVES_N == h) {
      const int row_l = (wave / TS::WAVES_N) * TS::WM + (lane & 31);
      const uint32_t key = (uint32_t)((row_l >> 1) & 7) << 4;   // rows row_l + 32 tm share it
      char* lb = fz + row_l * 128 + ((lane >> 5) << 3);
#pragma unroll
      for (int tm = 0; tm < TS::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TS::TN; ++tn)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            char* q0 = lb + tm * 32 * 128 + (((uint32_t)(tn * 4 + g) << 4) ^ key);
            Elem<uint16_t>::store4(reinterpret_cast<uint16_t*>(q0), ag[0][tm][tn][4 * g], ag[0][tm][tn][4 * g + 1], ag[0][tm][tn][4 * g + 2], ag[0][tm][tn][4 * g + 3]);
            Elem<uint16_t>::store4(reinterpret_cast<uint16_t*>(q0 + SM::A_BYTES), ay[0][tm][tn][4 * g], ay[0][tm][tn][4 * g + 1], ay[0][tm][tn][4 * g + 2], ay[0][tm][tn][4 * g + 3]);
            Elem<uint16_t>::store4(reinterpret_cast<uint16_t*>(q0 + SM::A_BYTES + SM::B_BYTES), ag[1][tm][tn][4 * g], ag[1][tm][tn][4 * g + 1], ag[1][tm][tn][4 * g + 2], ag[1][tm][tn][4 * g + 3]);
          }
    }
    __syncthreads();
    const char* st = smem + ((2 * nk + h) % STAGES) * SM::STAGE;
    const int j8 = threadIdx.x & 7;
    uint4 ui[2][3], uz[2][3];
    float l0[2], l1[2], l2[2];
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
      const int r = (threadIdx.x >> 3) + 64 * ps, m = m0 + r;
      const uint32_t o = (uint32_t)(r * 128 + ((j8 ^ ((r >> 1) & 7)) << 4));
      ui[ps][0] = *reinterpret_cast<const uint4*>(st + o);
      ui[ps][1] = *reinterpret_cast<const uint4*>(st + SM::A_BYTES + o);
      ui[ps][2] = *reinterpret_cast<const uint4*>(st + SM::A_BYTES + SM::B_BYTES + o);
      uz[ps][0] = *reinterpret_cast<const uint4*>(fz + o);
      uz[ps][1] = *reinterpret_cast<const uint4*>(fz + SM::A_BYTES + o);
      uz[ps][2] = *reinterpret_cast<const uint4*>(fz + SM::A_BYTES + SM::B_BYTES + o);
      const bool mv = m < p.T;
      l0[ps] = mv ? p.lr0[z * p.bslr + m] : 0.f;
      l1[ps] = mv ? p.lr1[z * p.bslr + m] : 0.f;
      l2[ps] = mv ? p.lr2[z * p.bslr + m] : 0.f;
    }
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
      const int r = (threadIdx.x >> 3) + 64 * ps, m = m0 + r;
      const bool mv = m < p.T;
      float gg[8], h2[8], dh[8], gz0[8], gz1[8], gz2[8], o0[8], o1[8], o2[8];
      unpack8(ui[ps][0], gg); unpack8(ui[ps][1], h2); unpack8(ui[ps][2], dh);
      unpack8(uz[ps][0], gz0); unpack8(uz[ps][1], gz1); unpack8(uz[ps][2], gz2);
      float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const SiluParts sp = silu_parts(gg[j]);
        const UpdatePointwise u = update_pointwise<uint16_t>(gg[j], h2[j], dh[j], sp);
        s0 += gz0[j] * u.dgpre; s1 += gz1[j] * u.hid; s2 += gz2[j] * u.dh2;
        const float ghid = gz1[j] * l1[ps], gdh2 = gz2[j] * l2[ps], gdg = gz0[j] * l0[ps];
        o0[j] = ghid * h2[j] * sp.d1 + gdh2 * dh[j] * sp.d1 + gdg * dh[j] * h2[j] * sp.d2;
        o1[j] = gdh2 * sp.silu + gdg * h2[j] * sp.d1;
        o2[j] = ghid * sp.silu + gdg * dh[j] * sp.d1;
      }
      // learning-rate gradients: the row's sum over this half's 64 columns (8 lanes), one partial per (row, half)
#pragma unroll
      for (int d = 1; d < 8; d <<= 1) {
        s0 += __shfl_xor(s0, d, 64); s1 += __shfl_xor(s1, d, 64); s2 += __shfl_xor(s2, d, 64);
      }
      if (mv) {
        const size_t o = off + (size_t)r * p.dh + h * 64 + j8 * 8;
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O0) + o) = pack8(o0);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O1) + o) = pack8(o1);
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(p.O2) + o) = pack8(o2);
        if (j8 == 0) {
          const size_t lo = (size_t)(by * TS::WAVES_N + h) * p.lrpart_stride + (size_t)z * p.Tcap + m;
          p.lrpart[0 * p.lrpart_mat_stride + lo] = s0;
          p.lrpart[1 * p.lrpart_mat_stride + lo] = s1;
          p.lrpart[2 * p.lrpart_mat_stride + lo] = s2;
        }
      }
    }
    if (h + 1 < halves) __syncthreads();   // the products of the next half go to the same place
  }
  // a half past the end of dh contributes nothing, but its slot of partial sums is read all the same
  for (int h = halves; h < TS::WAVES_N; ++h)
    if ((int)threadIdx.x < TS::BM && m0 + (int)threadIdx.x < p.T) {
      const size_t lo = (size_t)(by * TS::WAVES_N + h) * p.lrpart_stride + (size_t)z * p.Tcap + m0 + threadIdx.x;
      p.lrpart[0 * p.lrpart_mat_stride + lo] = 0.f;
      p.lrpart[1 * p.lrpart_mat_stride + lo] = 0.f;
      p.lrpart[2 * p.lrpart_mat_stride + lo] = 0.f;
    }
  LACT_TS(4);
}

// ------------------------------------------------------------------------------------------------
// k_token_reduce_dma: the three token-reduction GEMMs of one step (see k_token_reduce), both operands
// K-strided (tokens are the rows of every activation), fp32 partials per token split.
// ------------------------------------------------------------------------------------------------
struct TokenReduceDmaParams : TokenReduceParams {
  TileMap map;   // token splits, output tiles, 3 * batch
};
// One block of the reduction; `lin` is the block's linear index in the reduction's tile map.
template <class TS>
__device__ __forceinline__ void token_reduce_dma_block(const TokenReduceDmaParams& p, int lin, char* smem) {
  constexpr int STAGES = row_stages<TS>();
  using Pipe = DmaPipe<TS, 1, 2, STAGES, false, true>;
  int split, tile, bz;   // map: (splits, tiles, 3*nb)
  clear_words(p.prep_clear, lin == 0);
  if (!p.map.locate(lin, split, tile, bz)) return;
  const int j = bz / p.nb, ib = bz % p.nb;
  const TokenReduceJob& job = p.job[j];
  const int tiles_n = (job.N + TS::BN - 1) / TS::BN;
  const int m0 = (tile / tiles_n) * TS::BM, n0 = (tile % tiles_n) * TS::BN;
  if (m0 >= job.M) return;
  const int k_begin = split * p.split_len;
  const int klen = min(p.split_len, p.tokens - k_begin);
  DmaPhase<1> ph[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const TokenReduceTerm& tt = job.t[t < job.nterms ? t : 0];
    ph[t].a.base = reinterpret_cast<const uint16_t*>(tt.A) + ib * tt.bsA + (size_t)k_begin * tt.lda + m0;
    ph[t].a.ld = tt.lda; ph[t].a.rows = job.M - m0; ph[t].a.ks = 1;
    ph[t].b[0].base = reinterpret_cast<const uint16_t*>(tt.B) + ib * tt.bsB + (size_t)k_begin * tt.ldb + n0;
    ph[t].b[0].ld = tt.ldb; ph[t].b[0].rows = job.N - n0; ph[t].b[0].ks = 1;
    ph[t].nb = 1;
    // a token count that is not a multiple of 64 ends inside the last K-step of the last split
    ph[t].K = t < job.nterms ? (klen + DMA_BK - 1) / DMA_BK * DMA_BK : 0;
    ph[t].a.ktail = ph[t].b[0].ktail = klen % DMA_BK;
  }
  f32x16 acc[1][TS::TM][TS::TN];
  Pipe pipe(smem, ph);
  const bool loader = Pipe::is_loader();
  if (loader) {
    pipe.template load_all<Pipe::loads(1)>();
  } else {
    zero_acc<TS>(acc[0]);
    int step = 0;
    pipe.template run_phase<1, true, true>(ph[0].K / DMA_BK, step, acc);
    pipe.template run_phase<1, true, true>(ph[1].K / DMA_BK, step, acc);
  }
  __syncthreads();
  using ST = StageTile<TS, 4>;
  if (!loader) {
    char* lb = smem + ST::lane_base();
    LACT_FOR_QUADS(TS) ST::put4(lb, tm, tn, g, acc[0][tm][tn][4 * g], acc[0][tm][tn][4 * g + 1], acc[0][tm][tn][4 * g + 2], acc[0][tm][tn][4 * g + 3]);
  }
  __syncthreads();
  const size_t slot = (size_t)bz * p.mat_elems;
  if (p.prep_d_out) {   // forward update, one split: momentum, bf16 copy and its sum of squares right here
    const int r0 = ST::row0(), c0 = ST::col0();
    float ss = 0.f;
    if (ST::active() && n0 + c0 < job.N) {
      const char* src = smem + (r0 * ST::LD + c0) * 4;
      const size_t e0 = slot + (size_t)(m0 + r0) * job.N + n0 + c0, rstep = (size_t)ST::RPP * job.N;
      const float mb = (p.prep_m_prev && p.prep_mbar) ? p.prep_mbar[ib] : 0.f;
      float* ext = p.prep_m_ext[j] ? p.prep_m_ext[j] + (size_t)ib * p.mat_elems + (e0 - slot) : nullptr;
      float4 x4[ST::PASSES];
      if (p.prep_m_prev) {
#pragma unroll
        for (int ps = 0; ps < ST::PASSES; ++ps) {
          const int r = r0 + ps * ST::RPP;
          x4[ps] = (r < TS::BM && m0 + r < job.M) ? *reinterpret_cast<const float4*>(p.prep_m_prev + e0 + ps * rstep) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
      uint4 vg[8];
#pragma unroll
      for (int ps = 0; ps < ST::PASSES; ++ps) {
        if (ps % 8 == 0) {
#pragma unroll
          for (int g = 0; g < 8; ++g)
            if (ps + g < ST::PASSES) vg[g] = ST::read16(src, r0, ps + g);
        }
        const int r = r0 + ps * ST::RPP;
        if (r < TS::BM && m0 + r < job.M) {
          float4 v = __builtin_bit_cast(float4, vg[ps % 8]);
          v = make_float4(round_bf16(v.x), round_bf16(v.y), round_bf16(v.z), round_bf16(v.w));
          if (p.prep_m_prev) {   // product and sum rounded separately, as the reference's two tensor operations are
            v.x = __fadd_rn(v.x, __fmul_rn(x4[ps].x, mb)); v.y = __fadd_rn(v.y, __fmul_rn(x4[ps].y, mb));
            v.z = __fadd_rn(v.z, __fmul_rn(x4[ps].z, mb)); v.w = __fadd_rn(v.w, __fmul_rn(x4[ps].w, mb));
          }
          if (!p.prep_skip_d) *reinterpret_cast<float4*>(p.prep_d_out + e0 + ps * rstep) = v;
          if (ext) *reinterpret_cast<float4*>(ext + ps * rstep) = v;
          const float f0 = round_bf16(v.x), f1 = round_bf16(v.y), f2 = round_bf16(v.z), f3 = round_bf16(v.w);
          Elem<uint16_t>::store4(p.prep_g16 + e0 + ps * rstep, f0, f1, f2, f3);
          ss += f0 * f0 + f1 * f1 + f2 * f2 + f3 * f3;
        }
      }
    }
    ss = block_sum(ss, reinterpret_cast<float*>(smem));
    if (threadIdx.x == 0) p.prep_ss_part[(size_t)bz * p.map.gy + tile] = ss;
    return;
  }
  float* out = p.add_out ? p.add_out + slot : p.partial + (size_t)split * p.map.gz * p.mat_elems + slot;
  const int r0 = ST::row0(), c0 = ST::col0();
  if (ST::active() && n0 + c0 < job.N) {
    const char* src = smem + (r0 * ST::LD + c0) * 4;
    const size_t e0 = (size_t)(m0 + r0) * job.N + n0 + c0, rstep = (size_t)ST::RPP * job.N;
    float* dst = out + e0;
    const bool blend = p.add_out && p.add_in;
    float4 x4[ST::PASSES];
    if (blend) {
      const float* ain = p.add_in + slot + e0;
#pragma unroll
      for (int ps = 0; ps < ST::PASSES; ++ps) {
        const int r = r0 + ps * ST::RPP;
        x4[ps] = (r < TS::BM && m0 + r < job.M) ? *reinterpret_cast<const float4*>(ain + ps * rstep) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
    uint4 vg[8];
#pragma unroll
    for (int ps = 0; ps < ST::PASSES; ++ps) {
      if (ps % 8 == 0) {
#pragma unroll
        for (int g = 0; g < 8; ++g)
          if (ps + g < ST::PASSES) vg[g] = ST::read16(src, r0, ps + g);
      }
      const int r = r0 + ps * ST::RPP;
      if (r < TS::BM && m0 + r < job.M) {
        float4 v = __builtin_bit_cast(float4, vg[ps % 8]);
        if (blend) {
          v.x += p.coeff * x4[ps].x; v.y += p.coeff * x4[ps].y; v.z += p.coeff * x4[ps].z; v.w += p.coeff * x4[ps].w;
        }
        *reinterpret_cast<float4*>(dst) = v;
      }
      dst += rstep;
    }
  }
}

template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_token_reduce_dma(const TokenReduceDmaParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  token_reduce_dma_block<TS>(p, blockIdx.x, smem);
}

// The token reduction of an update's backward together with the two token-row GEMMs that read the same
// intermediates (dk: four terms, K-strided weights; dv: two terms): three independent pieces of work that, as
// launches of their own, each end in a round of blocks that leaves most compute units idle.  One grid, longest
// blocks first; every piece keeps its own tile map (the offsets are multiples of 8, so a block's XCD stays the
// one its map assumes).
struct TokenReduceRowsParams {
  TokenReduceDmaParams tr;
  RowGemmDmaParams<4> r4;
  RowGemmDmaParams<2> r2;
  int ntr, n4;   // blocks of the reduction and of the four-term GEMM
};
static_assert(sizeof(TokenReduceRowsParams) <= 4096, "kernel arguments must fit the 4 KiB argument segment");
template <class TS>
__global__ __launch_bounds__(DMA_THREADS) void k_token_reduce_rows_dma(const TokenReduceRowsParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int lin = blockIdx.x;
  if (lin < p.ntr) {
    token_reduce_dma_block<TS>(p.tr, lin, smem);
    return;
  }
  lin -= p.ntr;
  int bx, by, z;
  if (lin < p.n4) {
    if (!p.r4.map.locate(lin, bx, by, z)) return;
    row_gemm_tile<TS_ROW, 4, EPI_STORE, true, false>(p.r4, bx, by, z, smem);
    return;
  }
  lin -= p.n4;
  if (!p.r2.map.locate(lin, bx, by, z)) return;
  row_gemm_tile<TS_ROW, 2, EPI_STORE, false, false>(p.r2, bx, by, z, smem);
}

}  // namespace lact
