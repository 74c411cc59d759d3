// GEMM-shaped kernels of the TTT operation, all built on gemm_mainloop().
//
// Row layout throughout: activations are [tokens, feature] with the feature dimension contiguous;
// fast weights w0,w2 are [dh, d], w1 is [d, dh] (the reference's LLM layout,
// lact_llm/lact_model/ttt_operation.py:71-105).
#pragma once
#include "gemm_core.h"

namespace lact {

// ---- SwiGLU pointwise pieces -------------------------------------------------------------------
struct SiluParts {
  float sig, silu, d1, d2;  // sigmoid(x), x*sigmoid(x), silu'(x), silu''(x)
};
__device__ __forceinline__ SiluParts silu_parts(float x) {
  SiluParts p;
  p.sig = sigmoidf_(x);
  p.silu = x * p.sig;
  p.d1 = p.sig * (1.f + x * (1.f - p.sig));                        // ttt_operation.py:5-17
  p.d2 = p.sig * (1.f - p.sig) * (2.f + x * (1.f - 2.f * p.sig));  // derivative of the line above
  return p;
}

// ------------------------------------------------------------------------------------------------
// k_row_gemm: out[M, N] = epilogue( sum_terms A_t[M, K_t] * B_t ),  A K-contiguous (token rows),
// B either K-contiguous ([N, K]) or K-strided ([K, N]).  Grid (ceil(M/BM), ceil(N/BN), batch).
// ------------------------------------------------------------------------------------------------
struct RowGemmTerm {
  const void* A; int lda; long long bsA;
  const void* B; int ldb; long long bsB;
  int K;
};
enum { EPI_STORE = 0, EPI_AXPBY = 1, EPI_AXPBY_F32_DUAL = 2 };
template <int NT>
struct RowGemmParams {
  RowGemmTerm t[NT];
  int M, N;
  void* out; int ldo; long long bso;          // EPI_STORE, EPI_AXPBY: type T; DUAL: fp32
  int accumulate;                              // EPI_STORE only: out += result
  // EPI_STORE only, optional: out2 = round(alpha2 * round(acc)), type T, laid out like out (the product c*A that
  // ttt_operation.py:60 forms as a tensor of its own before the matmul)
  void* out2; float alpha2;
  // Every value that is a tensor in the reference's eager evaluation is rounded to its type T (identity for fp32):
  //   EPI_AXPBY:  out = round(round(alpha * round(acc)) + round(beta * aux))           (ttt_operation.py:59-61)
  //   DUAL:       out = alpha * round(acc) + beta * aux in fp32                        (:62 under autocast)
  //               round_out_bf16: round(round(alpha * round(acc)) + round(beta * aux)) (:62 without autocast)
  const void* aux; int ldaux; long long bsaux; // EPI_AXPBY: aux of type T; DUAL: fp32 aux
  float alpha, beta;
  void* out_c;                                 // DUAL: copy in type T, same ld/bs as out
  float* out_t; int transpose_mask; int nb;    // DUAL: optional fp32 copy; matrices whose (z / nb) bit is set are written transposed
  int round_out_bf16;                          // DUAL: round the fp32 result to bf16 (reference without autocast)
};

// X' = a X + B X (ttt_operation.py:62): `prod` = alpha * round(acc), `ax` = beta * aux.  Without autocast both are bf16
// tensors and so is their sum.
__device__ __forceinline__ float dual_blend(float prod, float ax, int plain_bf16) {
  return plain_bf16 ? round_bf16(round_bf16(prod) + round_bf16(ax)) : __fadd_rn(ax, prod);
}

template <typename T, class TS, bool B_KC, int NT, int EPI>
__global__ __launch_bounds__(TS::THREADS) void k_row_gemm(const RowGemmParams<NT> p) {
  __shared__ __attribute__((aligned(16))) char smem[GemmSmem<T, TS>::BYTES];
  const int m0 = blockIdx.x * TS::BM, n0 = blockIdx.y * TS::BN, z = blockIdx.z;
  f32x16 acc[TS::TM][TS::TN];
  zero_acc<TS>(acc);
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const T* A = reinterpret_cast<const T*>(p.t[t].A) + z * p.t[t].bsA + (size_t)m0 * p.t[t].lda;
    const T* B = reinterpret_cast<const T*>(p.t[t].B) + z * p.t[t].bsB + (B_KC ? (size_t)n0 * p.t[t].ldb : (size_t)n0);
    gemm_mainloop<T, TS, true, B_KC>(acc, A, p.t[t].lda, p.M - m0, B, p.t[t].ldb, p.N - n0, p.t[t].K, smem);
  }
  LACT_FOR_QUADS(TS) {
    const int m = m0 + quad_m<TS>(tm), n = n0 + quad_n<TS>(tn, g);
    if (m >= p.M || n >= p.N) continue;
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = acc[tm][tn][4 * g + j];
    if (EPI == EPI_STORE) {
      T* o = reinterpret_cast<T*>(p.out) + z * p.bso + (size_t)m * p.ldo + n;
      if (p.accumulate) {
        float old[4];
        Elem<T>::load4(o, old);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += old[j];
      }
      Elem<T>::store4(o, v[0], v[1], v[2], v[3]);
      if (p.out2) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = p.alpha2 * Elem<T>::rnd(v[j]);
        Elem<T>::store4(reinterpret_cast<T*>(p.out2) + z * p.bso + (size_t)m * p.ldo + n, v[0], v[1], v[2], v[3]);
      }
    } else if (EPI == EPI_AXPBY) {
      float a[4];
      Elem<T>::load4(reinterpret_cast<const T*>(p.aux) + z * p.bsaux + (size_t)m * p.ldaux + n, a);
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = Elem<T>::rnd(p.alpha * Elem<T>::rnd(v[j])) + Elem<T>::rnd(p.beta * a[j]);
      Elem<T>::store4(reinterpret_cast<T*>(p.out) + z * p.bso + (size_t)m * p.ldo + n, v[0], v[1], v[2], v[3]);
    } else {
      float a[4];
      Elem<float>::load4(reinterpret_cast<const float*>(p.aux) + z * p.bsaux + (size_t)m * p.ldaux + n, a);
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = dual_blend(__fmul_rn(p.alpha, Elem<T>::rnd(v[j])), __fmul_rn(p.beta, a[j]), p.round_out_bf16);
      const size_t off = z * p.bso + (size_t)m * p.ldo + n;
      if (p.out) Elem<float>::store4(reinterpret_cast<float*>(p.out) + off, v[0], v[1], v[2], v[3]);
      if (p.out_c) Elem<T>::store4(reinterpret_cast<T*>(p.out_c) + off, v[0], v[1], v[2], v[3]);
      if (p.out_t) {
        float* o = p.out_t + z * p.bso;
        if ((p.transpose_mask >> (z / p.nb)) & 1) {
#pragma unroll
          for (int j = 0; j < 4; ++j) o[(size_t)(n + j) * p.M + m] = v[j];
        } else {
          Elem<float>::store4(o + (size_t)m * p.ldo + n, v[0], v[1], v[2], v[3]);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Hidden-layer kernels: token tile x hidden tile, several accumulators sharing the token tile.
// Grid (ceil(tokens/BM), ceil(dh/BN), b).
// ------------------------------------------------------------------------------------------------
struct HiddenParams {
  int T, d, dh;                    // tokens in this step, feature dim, hidden dim
  const void* X; int ldx; long long bsx;   // q (apply) or k (update)            [T, d]
  const void* Y; int ldy; long long bsy;   // v (update) or upstream grad (apply backward) [T, d]
  const void* W0; const void* W1; const void* W2; long long bsw;  // compute copies, type T
  const float* lr0; const float* lr1; const float* lr2; long long bslr;  // [b, *] already offset to this step
  // gradients of the fast-weight gradients (backward of the update): G0,G2 [dh,d], G1 [d,dh], type T
  const void* G0; const void* G1; const void* G2;
  void* O0; void* O1; void* O2; void* O3; void* O4; void* O5;  // [b, T, dh] outputs, type T
  void* O6; void* O7;               // update forward: lr-scaled copies of O0 and O2 kept for the backward (nullable)
  long long bso;
  // update backward from kept pre-activations: I0 = k W0^T, I1 = k W2^T, I2 = v W1 as the forward rounded them
  const void* I0; const void* I1; const void* I2; long long bsi;
  float* lrpart; long long lrpart_stride;  // partial row sums: [3][nparts][b*Tcap]; stride between parts
  long long lrpart_mat_stride;
  int Tcap;
};

// apply forward:  O0 = silu(X W0^T) * (X W2^T)                       (ttt_operation.py:141-143)
template <typename T, class TS>
__global__ __launch_bounds__(TS::THREADS) void k_apply_hidden(const HiddenParams p) {
  __shared__ __attribute__((aligned(16))) char smem[GemmSmem<T, TS>::BYTES];
  const int m0 = blockIdx.x * TS::BM, n0 = blockIdx.y * TS::BN, z = blockIdx.z;
  const T* X = reinterpret_cast<const T*>(p.X) + z * p.bsx + (size_t)m0 * p.ldx;
  const T* W0 = reinterpret_cast<const T*>(p.W0) + z * p.bsw + (size_t)n0 * p.d;
  const T* W2 = reinterpret_cast<const T*>(p.W2) + z * p.bsw + (size_t)n0 * p.d;
  f32x16 a0[TS::TM][TS::TN], a2[TS::TM][TS::TN];
  zero_acc<TS>(a0);
  zero_acc<TS>(a2);
  gemm_mainloop<T, TS, true, true>(a0, X, p.ldx, p.T - m0, W0, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, true>(a2, X, p.ldx, p.T - m0, W2, p.d, p.dh - n0, p.d, smem);
  LACT_FOR_QUADS(TS) {
    const int m = m0 + quad_m<TS>(tm), n = n0 + quad_n<TS>(tn, g);
    if (m >= p.T || n >= p.dh) continue;
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float y0 = Elem<T>::rnd(a0[tm][tn][4 * g + j]), y2 = Elem<T>::rnd(a2[tm][tn][4 * g + j]);
      v[j] = Elem<T>::rnd(y0 * sigmoidf_(y0)) * y2;
    }
    Elem<T>::store4(reinterpret_cast<T*>(p.O0) + z * p.bso + (size_t)m * p.dh + n, v[0], v[1], v[2], v[3]);
  }
}

// Shared by the update forward and its backward: what the three lr-scaled GEMM operands are.
struct UpdatePointwise {
  float hid, dh2, dgpre;
};
template <typename T>
__device__ __forceinline__ UpdatePointwise update_pointwise(float g, float h2, float dh, const SiluParts& s) {
  UpdatePointwise u;
  const float sg = Elem<T>::rnd(s.silu);
  u.hid = Elem<T>::rnd(sg * h2);                       // ttt_operation.py:150
  u.dh2 = Elem<T>::rnd(dh * sg);                       // :155
  // silu_backprop(dhidden * hidden_before_mul, gate_before_act), :157-158 with :15-16 evaluated operation by
  // operation on tensors of type T as eager PyTorch does: dy * sigma * (1 + x * (1 - sigma))
  const float sb = Elem<T>::rnd(s.sig), dg = Elem<T>::rnd(dh * h2);
  const float t1 = Elem<T>::rnd(dg * sb);
  const float t4 = Elem<T>::rnd(1.f + Elem<T>::rnd(g * Elem<T>::rnd(1.f - sb)));
  u.dgpre = Elem<T>::rnd(t1 * t4);
  return u;
}

// update forward:  O0 = dgate_before_act, O1 = hidden * lr1, O2 = dhidden_before_mul
// (ttt_operation.py:147-168: lr1 scales the hidden-side operand of dw1, lr0 and lr2 scale k -- see k_lr_scale_rows).
template <typename T, class TS>
__global__ __launch_bounds__(TS::THREADS) void k_update_hidden(const HiddenParams p) {
  __shared__ __attribute__((aligned(16))) char smem[GemmSmem<T, TS>::BYTES];
  const int m0 = blockIdx.x * TS::BM, n0 = blockIdx.y * TS::BN, z = blockIdx.z;
  const T* X = reinterpret_cast<const T*>(p.X) + z * p.bsx + (size_t)m0 * p.ldx;
  const T* Y = reinterpret_cast<const T*>(p.Y) + z * p.bsy + (size_t)m0 * p.ldy;
  const T* W0 = reinterpret_cast<const T*>(p.W0) + z * p.bsw + (size_t)n0 * p.d;
  const T* W2 = reinterpret_cast<const T*>(p.W2) + z * p.bsw + (size_t)n0 * p.d;
  const T* W1 = reinterpret_cast<const T*>(p.W1) + z * p.bsw + n0;  // [d, dh]: K-strided for V*W1
  f32x16 a0[TS::TM][TS::TN], a2[TS::TM][TS::TN], a1[TS::TM][TS::TN];
  zero_acc<TS>(a0);
  zero_acc<TS>(a2);
  zero_acc<TS>(a1);
  gemm_mainloop<T, TS, true, true>(a0, X, p.ldx, p.T - m0, W0, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, true>(a2, X, p.ldx, p.T - m0, W2, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, false>(a1, Y, p.ldy, p.T - m0, W1, p.dh, p.dh - n0, p.d, smem);
  LACT_FOR_QUADS(TS) {
    const int m = m0 + quad_m<TS>(tm), n = n0 + quad_n<TS>(tn, g);
    if (m >= p.T || n >= p.dh) continue;
    const float l1 = p.lr1[z * p.bslr + m];
    float z0[4], z1[4], z2[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float gg = Elem<T>::rnd(a0[tm][tn][4 * g + j]), h2 = Elem<T>::rnd(a2[tm][tn][4 * g + j]);
      const float dh = Elem<T>::rnd(a1[tm][tn][4 * g + j]);
      const UpdatePointwise u = update_pointwise<T>(gg, h2, dh, silu_parts(gg));
      z0[j] = u.dgpre;
      z1[j] = u.hid * l1;
      z2[j] = u.dh2;
    }
    const size_t off = z * p.bso + (size_t)m * p.dh + n;
    Elem<T>::store4(reinterpret_cast<T*>(p.O0) + off, z0[0], z0[1], z0[2], z0[3]);
    Elem<T>::store4(reinterpret_cast<T*>(p.O1) + off, z1[0], z1[1], z1[2], z1[3]);
    Elem<T>::store4(reinterpret_cast<T*>(p.O2) + off, z2[0], z2[1], z2[2], z2[3]);
  }
}

// kl0 = T(k * lr0), kl2 = T(k * lr2): the token-major operands of the dw0 and dw2 reductions.  The reference scales
// k by the per-token rate and casts the product before the matmul (ttt_operation.py:167-168, lact_ttt.py:122-126),
// so the rounding has to happen on this side of the contraction.  k: [b, tokens, d] with row / batch strides;
// outputs contiguous [b][tokens][d] with batch stride bso.  Grid (ceil(tokens * d / 4 / 256), b).
template <typename T>
__global__ void k_lr_scale_rows(const T* k, int ld, long long bs, const float* lr0, const float* lr2, long long bslr,
                                int tokens, int d, T* o0, T* o2, long long bso) {
  const long long e = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int z = blockIdx.y;
  if (e >= (long long)tokens * d) return;
  const int t = (int)(e / d), c = (int)(e % d);
  float v[4];
  Elem<T>::load4(k + z * bs + (size_t)t * ld + c, v);
  const float l0 = lr0[z * bslr + t], l2 = lr2[z * bslr + t];
  Elem<T>::store4(o0 + z * bso + e, v[0] * l0, v[1] * l0, v[2] * l0, v[3] * l0);
  Elem<T>::store4(o2 + z * bso + e, v[0] * l2, v[1] * l2, v[2] * l2, v[3] * l2);
}

// Row sums over the hidden dimension of a per-thread partial: lanes l and l^32 hold the same token.
// Each wave then owns one partial per token; the slot index is (hidden tile, wave column).
template <class TS>
__device__ __forceinline__ void store_row_partials(const HiddenParams& p, int which, int tm, int m, int z, float v, int ytile) {
  v += __shfl_xor(v, 32, 64);
  if ((threadIdx.x & 63) < 32 && m < p.T) {
    const int slot = ytile * TS::WAVES_N + ((threadIdx.x >> 6) % TS::WAVES_N);
    p.lrpart[which * p.lrpart_mat_stride + slot * p.lrpart_stride + (size_t)z * p.Tcap + m] = v;
  }
}

// apply backward, hidden stage:  O0 = hidden (recomputed), O1 = d/d(X W0^T), O2 = d/d(X W2^T)
// with Y = upstream gradient of the apply output  (lact_triton_kernels/lact_swiglu_ffn.py:57-65).
template <typename T, class TS>
__global__ __launch_bounds__(TS::THREADS) void k_apply_bwd_hidden(const HiddenParams p) {
  __shared__ __attribute__((aligned(16))) char smem[GemmSmem<T, TS>::BYTES];
  const int m0 = blockIdx.x * TS::BM, n0 = blockIdx.y * TS::BN, z = blockIdx.z;
  const T* X = reinterpret_cast<const T*>(p.X) + z * p.bsx + (size_t)m0 * p.ldx;
  const T* Y = reinterpret_cast<const T*>(p.Y) + z * p.bsy + (size_t)m0 * p.ldy;
  const T* W0 = reinterpret_cast<const T*>(p.W0) + z * p.bsw + (size_t)n0 * p.d;
  const T* W2 = reinterpret_cast<const T*>(p.W2) + z * p.bsw + (size_t)n0 * p.d;
  const T* W1 = reinterpret_cast<const T*>(p.W1) + z * p.bsw + n0;
  f32x16 a0[TS::TM][TS::TN], a2[TS::TM][TS::TN], a1[TS::TM][TS::TN];
  zero_acc<TS>(a0);
  zero_acc<TS>(a2);
  zero_acc<TS>(a1);
  gemm_mainloop<T, TS, true, true>(a0, X, p.ldx, p.T - m0, W0, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, true>(a2, X, p.ldx, p.T - m0, W2, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, false>(a1, Y, p.ldy, p.T - m0, W1, p.dh, p.dh - n0, p.d, smem);
  LACT_FOR_QUADS(TS) {
    const int m = m0 + quad_m<TS>(tm), n = n0 + quad_n<TS>(tn, g);
    if (m >= p.T || n >= p.dh) continue;
    float hq[4], gy0[4], gy2[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float y0 = Elem<T>::rnd(a0[tm][tn][4 * g + j]), y2 = Elem<T>::rnd(a2[tm][tn][4 * g + j]);
      const float gh = Elem<T>::rnd(a1[tm][tn][4 * g + j]);
      const SiluParts s = silu_parts(y0);
      const float sg = Elem<T>::rnd(s.silu);
      hq[j] = sg * y2;
      gy0[j] = Elem<T>::rnd(gh * y2) * s.d1;   // the gradient of the gate is a tensor of type T before silu's backward
      gy2[j] = gh * sg;
    }
    const size_t off = z * p.bso + (size_t)m * p.dh + n;
    Elem<T>::store4(reinterpret_cast<T*>(p.O0) + off, hq[0], hq[1], hq[2], hq[3]);
    Elem<T>::store4(reinterpret_cast<T*>(p.O1) + off, gy0[0], gy0[1], gy0[2], gy0[3]);
    Elem<T>::store4(reinterpret_cast<T*>(p.O2) + off, gy2[0], gy2[1], gy2[2], gy2[3]);
  }
}

// update backward, hidden stage (second order; lact_triton_kernels/lact_fw_grad.py:82-119,179-260).
// Recomputes gate / hidden / dhidden, forms the gradients with respect to the three lr-scaled
// operands (K G0^T, V G1, K G2^T) and emits
//   O0 = d/d gate_before_act, O1 = d/d dhidden, O2 = d/d hidden_before_mul,
//   O3 = dgate_before_act*lr0, O4 = hidden*lr1, O5 = dhidden_before_mul*lr2 (recomputed operands)
// plus per-token partial sums of the lr gradients.
template <typename T, class TS>
__global__ __launch_bounds__(TS::THREADS) void k_update_bwd_hidden(const HiddenParams p) {
  __shared__ __attribute__((aligned(16))) char smem[GemmSmem<T, TS>::BYTES];
  const int m0 = blockIdx.x * TS::BM, n0 = blockIdx.y * TS::BN, z = blockIdx.z;
  const T* X = reinterpret_cast<const T*>(p.X) + z * p.bsx + (size_t)m0 * p.ldx;
  const T* Y = reinterpret_cast<const T*>(p.Y) + z * p.bsy + (size_t)m0 * p.ldy;
  const T* W0 = reinterpret_cast<const T*>(p.W0) + z * p.bsw + (size_t)n0 * p.d;
  const T* W2 = reinterpret_cast<const T*>(p.W2) + z * p.bsw + (size_t)n0 * p.d;
  const T* W1 = reinterpret_cast<const T*>(p.W1) + z * p.bsw + n0;
  const T* G0 = reinterpret_cast<const T*>(p.G0) + z * p.bsw + (size_t)n0 * p.d;
  const T* G2 = reinterpret_cast<const T*>(p.G2) + z * p.bsw + (size_t)n0 * p.d;
  const T* G1 = reinterpret_cast<const T*>(p.G1) + z * p.bsw + n0;
  f32x16 a0[TS::TM][TS::TN], a2[TS::TM][TS::TN], a1[TS::TM][TS::TN];
  f32x16 b0[TS::TM][TS::TN], b2[TS::TM][TS::TN], b1[TS::TM][TS::TN];
  zero_acc<TS>(a0); zero_acc<TS>(a2); zero_acc<TS>(a1);
  zero_acc<TS>(b0); zero_acc<TS>(b2); zero_acc<TS>(b1);
  gemm_mainloop<T, TS, true, true>(a0, X, p.ldx, p.T - m0, W0, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, true>(a2, X, p.ldx, p.T - m0, W2, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, true>(b0, X, p.ldx, p.T - m0, G0, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, true>(b2, X, p.ldx, p.T - m0, G2, p.d, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, false>(a1, Y, p.ldy, p.T - m0, W1, p.dh, p.dh - n0, p.d, smem);
  gemm_mainloop<T, TS, true, false>(b1, Y, p.ldy, p.T - m0, G1, p.dh, p.dh - n0, p.d, smem);
#pragma unroll
  for (int tm = 0; tm < TS::TM; ++tm) {
    const int m = m0 + quad_m<TS>(tm);
    const bool mv = m < p.T;
    const float l0 = mv ? p.lr0[z * p.bslr + m] : 0.f, l1 = mv ? p.lr1[z * p.bslr + m] : 0.f;
    const float l2 = mv ? p.lr2[z * p.bslr + m] : 0.f;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int tn = 0; tn < TS::TN; ++tn)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + quad_n<TS>(tn, g);
        if (!mv || n >= p.dh) continue;
        float o0[4], o1[4], o2[4], o3[4], o4[4], o5[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float gg = Elem<T>::rnd(a0[tm][tn][4 * g + j]), h2 = Elem<T>::rnd(a2[tm][tn][4 * g + j]);
          const float dh = Elem<T>::rnd(a1[tm][tn][4 * g + j]);
          const float gz0 = Elem<T>::rnd(b0[tm][tn][4 * g + j]), gz2 = Elem<T>::rnd(b2[tm][tn][4 * g + j]);
          const float gz1 = Elem<T>::rnd(b1[tm][tn][4 * g + j]);
          const SiluParts s = silu_parts(gg);
          const UpdatePointwise u = update_pointwise<T>(gg, h2, dh, s);
          s0 += gz0 * u.dgpre;
          s1 += gz1 * u.hid;
          s2 += gz2 * u.dh2;
          const float ghid = gz1 * l1, gdh2 = gz2 * l2, gdg = gz0 * l0;
          o0[j] = ghid * h2 * s.d1 + gdh2 * dh * s.d1 + gdg * dh * h2 * s.d2;   // d gate_before_act
          o1[j] = gdh2 * s.silu + gdg * h2 * s.d1;                             // d dhidden
          o2[j] = ghid * s.silu + gdg * dh * s.d1;                             // d hidden_before_mul
          o3[j] = u.dgpre * l0;
          o4[j] = u.hid * l1;
          o5[j] = u.dh2 * l2;
        }
        const size_t off = z * p.bso + (size_t)m * p.dh + n;
        Elem<T>::store4(reinterpret_cast<T*>(p.O0) + off, o0[0], o0[1], o0[2], o0[3]);
        Elem<T>::store4(reinterpret_cast<T*>(p.O1) + off, o1[0], o1[1], o1[2], o1[3]);
        Elem<T>::store4(reinterpret_cast<T*>(p.O2) + off, o2[0], o2[1], o2[2], o2[3]);
        Elem<T>::store4(reinterpret_cast<T*>(p.O3) + off, o3[0], o3[1], o3[2], o3[3]);
        Elem<T>::store4(reinterpret_cast<T*>(p.O4) + off, o4[0], o4[1], o4[2], o4[3]);
        Elem<T>::store4(reinterpret_cast<T*>(p.O5) + off, o5[0], o5[1], o5[2], o5[3]);
      }
    store_row_partials<TS>(p, 0, tm, m, z, s0, blockIdx.y);
    store_row_partials<TS>(p, 1, tm, m, z, s1, blockIdx.y);
    store_row_partials<TS>(p, 2, tm, m, z, s2, blockIdx.y);
  }
}

// ------------------------------------------------------------------------------------------------
// k_token_reduce: the three token-reduction GEMMs of one step, split over tokens.
//   job j, batch ib:  P[j][ib][M_j, N_j] = sum over terms  A_t[tokens, M_j]^T * B_t[tokens, N_j]
// Both operands K-strided.  Grid (max tiles, splits, 3*b); fp32 partials [split][3*b][M*N].
// ------------------------------------------------------------------------------------------------
struct TokenReduceTerm {
  const void* A; int lda; long long bsA;
  const void* B; int ldb; long long bsB;
};
struct TokenReduceJob {
  TokenReduceTerm t[2];
  int nterms, M, N;
};
struct TokenReduceParams {
  TokenReduceJob job[3];
  int nb, tokens, split_len;   // split_len: tokens per split (multiple of 32)
  float* partial; long long mat_elems;
  // single split only (asynchronous-copy kernel): out = coeff*add_in + result written here instead of a partial
  float* add_out; const float* add_in; float coeff;
  // single split only, forward update: what k_momentum_prep would do with the result, done by the epilogue --
  // d_out = round_bf16(result) + m_prev * mbar[batch] (fp32 momentum state), its bf16 copy g16 in the same
  // layout, and the sum of squares of that copy per block in ss_part[matrix][tile]
  float* prep_d_out; const float* prep_m_prev; const float* prep_mbar; uint16_t* prep_g16; float* prep_ss_part;
  float* prep_m_ext[3];    // caller's momentum outputs [b][elems] per matrix kind (same values as d_out), each nullable
  int prep_skip_d;         // nothing reads d_out after this update (it stays the switch of the folded epilogue): not stored
  ClearWords prep_clear;   // barrier lines of the fused Newton-Schulz kernel that follows (cleared by the first block)
};

template <typename T, class TS>
__global__ __launch_bounds__(TS::THREADS) void k_token_reduce(const TokenReduceParams p) {
  __shared__ __attribute__((aligned(16))) char smem[GemmSmem<T, TS>::BYTES];
  const int j = blockIdx.z / p.nb, ib = blockIdx.z % p.nb;
  const TokenReduceJob& job = p.job[j];
  const int tiles_n = (job.N + TS::BN - 1) / TS::BN;
  const int m0 = (blockIdx.x / tiles_n) * TS::BM, n0 = (blockIdx.x % tiles_n) * TS::BN;
  if (m0 >= job.M) return;
  const int k_begin = blockIdx.y * p.split_len;
  const int klen = min(p.split_len, p.tokens - k_begin);
  f32x16 acc[TS::TM][TS::TN];
  zero_acc<TS>(acc);
  for (int t = 0; t < job.nterms; ++t) {
    const T* A = reinterpret_cast<const T*>(job.t[t].A) + ib * job.t[t].bsA + (size_t)k_begin * job.t[t].lda + m0;
    const T* B = reinterpret_cast<const T*>(job.t[t].B) + ib * job.t[t].bsB + (size_t)k_begin * job.t[t].ldb + n0;
    gemm_mainloop<T, TS, false, false>(acc, A, job.t[t].lda, job.M - m0, B, job.t[t].ldb, job.N - n0, klen, smem);
  }
  float* out = p.partial + ((size_t)blockIdx.y * gridDim.z + blockIdx.z) * p.mat_elems;
  LACT_FOR_QUADS(TS) {
    const int m = m0 + quad_m<TS>(tm), n = n0 + quad_n<TS>(tn, g);
    if (m >= job.M || n >= job.N) continue;
    Elem<float>::store4(out + (size_t)m * job.N + n, acc[tm][tn][4 * g], acc[tm][tn][4 * g + 1], acc[tm][tn][4 * g + 2],
                        acc[tm][tn][4 * g + 3]);
  }
}

}  // namespace lact
