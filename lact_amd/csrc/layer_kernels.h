// Pre- and post-processing of the layer classes around the TTT operation, one pass over the data each:
//
//   pre :  qkv [B, L, 3, H, hd]  ->  q, k, v [(B H), L, hd]     silu, per-head L2 norm of q and k, head layout
//          (bidirectional_lact_layer.py:231-244, causal_lact_with_sliding_window_attn.py:313-322)
//   lr  :  raw [B, L, H, 3] -> lr0, lr1, lr2 [(B H), L]          softplus(raw + inverse-softplus(base lr))
//          momentum raw [B, L, H] -> [(B H), L]                  sigmoid
//          (bidirectional_lact_layer.py:248-256, causal_...:326-345)
//   post:  o [(B H), L, hd] -> y [B, L, H*hd]                    per-head RMSNorm (affine), optional silu gate per
//          token and head, head layout  (bidirectional_lact_layer.py:268-270, causal_...:351-357)
//
// and their backward passes.  One wave per (token, head) row of hd elements; 16 bytes per lane.
// Element type T = uint16_t (bf16) or float; all statistics in fp32.
#pragma once
#include "common.h"

namespace lact {

struct LayerGeom {
  int B, L, H, hd;
  __device__ __forceinline__ long long rows() const { return (long long)B * L * H; }
};

__device__ __forceinline__ float silu_f(float x) { return x * sigmoidf_(x); }
__device__ __forceinline__ float silu_grad_f(float x) {
  const float s = sigmoidf_(x);
  return s * (1.f + x * (1.f - s));
}

constexpr int LAYER_VEC_MAX = 4;   // a lane keeps up to 4 x 4 elements of its row (hd <= 1024)

// ---- pre ------------------------------------------------------------------------------------------
struct LayerPreParams {
  LayerGeom g;
  int l2norm;                 // L2-normalise q and k
  const void* qkv;            // [B, L, 3, H, hd]
  void* out[3];               // q, k, v  [(B H), L, hd]
  // backward
  const void* dout[3];
  void* dqkv;
};

// Grid: ceil(rows / 4) blocks of 256 threads, one wave per (b, l, h); the wave handles q, k and v of its row.
template <typename T, bool BWD>
__global__ __launch_bounds__(256) void k_layer_pre(const LayerPreParams p) {
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= p.g.rows()) return;
  const int h = (int)(row % p.g.H);
  const long long bl = row / p.g.H;            // b*L + l
  const int l = (int)(bl % p.g.L);
  const long long b = bl / p.g.L;
  const int hd = p.g.hd;
#pragma unroll
  for (int which = 0; which < 3; ++which) {
    const size_t si = ((size_t)(bl * 3 + which) * p.g.H + h) * hd;
    const size_t oi = ((size_t)(b * p.g.H + h) * p.g.L + l) * hd;
    const T* src = reinterpret_cast<const T*>(p.qkv) + si;
    const bool norm = p.l2norm && which < 2;
    float x[LAYER_VEC_MAX][4], y[LAYER_VEC_MAX][4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < LAYER_VEC_MAX; ++i) {
      const int c = lane * 4 + i * 256;
      if (c < hd) {
        Elem<T>::load4(src + c, x[i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          y[i][j] = Elem<T>::rnd(silu_f(x[i][j]));       // silu output is a tensor of type T in the reference
          ss += y[i][j] * y[i][j];
        }
      }
    }
    float n = 0.f;
    if (norm) n = sqrtf(wave_sum(ss));
    const float inv = norm ? 1.f / (n + 1e-5f) : 1.f;
    if (!BWD) {
      T* dst = reinterpret_cast<T*>(p.out[which]) + oi;
#pragma unroll
      for (int i = 0; i < LAYER_VEC_MAX; ++i) {
        const int c = lane * 4 + i * 256;
        if (c < hd) Elem<T>::store4(dst + c, y[i][0] * inv, y[i][1] * inv, y[i][2] * inv, y[i][3] * inv);
      }
    } else {
      // z = y / (n + eps):  dy = dz / (n + eps) - y <dz, y> / (n (n + eps)^2);  dx = dy silu'(x)
      const T* dz = reinterpret_cast<const T*>(p.dout[which]) + oi;
      float g[LAYER_VEC_MAX][4];
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < LAYER_VEC_MAX; ++i) {
        const int c = lane * 4 + i * 256;
        if (c < hd) {
          Elem<T>::load4(dz + c, g[i]);
#pragma unroll
          for (int j = 0; j < 4; ++j) dot += g[i][j] * y[i][j];
        }
      }
      float c1 = 0.f;
      if (norm) {
        dot = wave_sum(dot);
        c1 = n > 0.f ? dot / (n * (n + 1e-5f) * (n + 1e-5f)) : 0.f;
      }
      T* dx = reinterpret_cast<T*>(p.dqkv) + si;
#pragma unroll
      for (int i = 0; i < LAYER_VEC_MAX; ++i) {
        const int c = lane * 4 + i * 256;
        if (c < hd) {
          float o[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = (g[i][j] * inv - y[i][j] * c1) * silu_grad_f(x[i][j]);
          Elem<T>::store4(dx + c, o[0], o[1], o[2], o[3]);
        }
      }
    }
  }
}

// ---- learning rates and momentum ------------------------------------------------------------------
struct LayerLrParams {
  LayerGeom g;
  float base_lr_inv;
  const float* lr_raw;        // [B, L, H, 3], or [B, L, 3, H] when rates_major
  int rates_major;
  float* lr[3];               // [(B H), L]
  const float* mom_raw;       // [B, L, H] or null
  float* mom;                 // [(B H), L]
  // backward
  const float* dlr[3]; const float* dmom;
  float* dlr_raw; float* dmom_raw;
};
template <bool BWD>
__global__ void k_layer_lr(const LayerLrParams p) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;   // over (b, l, h)
  if (i >= p.g.rows()) return;
  const int h = (int)(i % p.g.H);
  const long long bl = i / p.g.H;
  const int l = (int)(bl % p.g.L);
  const long long b = bl / p.g.L;
  const size_t o = (size_t)(b * p.g.H + h) * p.g.L + l;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    const long long ri = p.rates_major ? (bl * 3 + s) * p.g.H + h : i * 3 + s;
    const float x = p.lr_raw[ri] + p.base_lr_inv;
    if (!BWD) p.lr[s][o] = x > 20.f ? x : log1pf(__expf(x));          // softplus (threshold as in torch)
    else p.dlr_raw[ri] = p.dlr[s] ? p.dlr[s][o] * (x > 20.f ? 1.f : sigmoidf_(x)) : 0.f;
  }
  if (p.mom_raw) {
    const float s = sigmoidf_(p.mom_raw[i]);
    if (!BWD) p.mom[o] = s;
    else p.dmom_raw[i] = p.dmom ? p.dmom[o] * s * (1.f - s) : 0.f;
  }
}

// ---- post -----------------------------------------------------------------------------------------
struct LayerPostParams {
  LayerGeom g;
  float eps;
  int use_norm;
  const void* o;              // [(B H), L, hd]
  const float* w;             // [hd] RMSNorm weight (null = ones)
  const void* gate_raw;       // [B, L, H] type T, or null: y *= silu(gate_raw)
  void* y;                    // [B, L, H*hd]
  // backward
  const void* dy; void* d_o; void* dgate_raw;
  float* dw_part;             // [gridDim.x * 4][hd] partial sums of the weight gradient, or null
};
// Backward: each wave walks rows row0, row0 + stride, ... so that its partial weight gradient stays in registers.
template <typename T, bool BWD>
__global__ __launch_bounds__(256) void k_layer_post(const LayerPostParams p) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long long nwaves = (long long)gridDim.x * 4;
  const int hd = p.g.hd;
  float wv[LAYER_VEC_MAX][4], dwacc[LAYER_VEC_MAX][4];
#pragma unroll
  for (int i = 0; i < LAYER_VEC_MAX; ++i) {
    const int c = lane * 4 + i * 256;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      wv[i][j] = (p.w && c < hd) ? p.w[c + j] : 1.f;
      dwacc[i][j] = 0.f;
    }
  }
  for (long long row = (long long)blockIdx.x * 4 + wave; row < p.g.rows(); row += nwaves) {
    const int h = (int)(row % p.g.H);
    const long long bl = row / p.g.H;
    const int l = (int)(bl % p.g.L);
    const long long b = bl / p.g.L;
    const size_t oi = ((size_t)(b * p.g.H + h) * p.g.L + l) * hd;
    const size_t yi = ((size_t)bl * p.g.H + h) * hd;
    const T* src = reinterpret_cast<const T*>(p.o) + oi;
    float x[LAYER_VEC_MAX][4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < LAYER_VEC_MAX; ++i) {
      const int c = lane * 4 + i * 256;
      if (c < hd) {
        Elem<T>::load4(src + c, x[i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) ss += x[i][j] * x[i][j];
      }
    }
    float rstd = 1.f;
    if (p.use_norm) rstd = rsqrtf(wave_sum(ss) / (float)hd + p.eps);
    float graw = 0.f, gate = 1.f;
    if (p.gate_raw) {
      graw = Elem<T>::load(reinterpret_cast<const T*>(p.gate_raw) + bl * p.g.H + h);
      gate = Elem<T>::rnd(silu_f(graw));
    }
    if (!BWD) {
      T* dst = reinterpret_cast<T*>(p.y) + yi;
#pragma unroll
      for (int i = 0; i < LAYER_VEC_MAX; ++i) {
        const int c = lane * 4 + i * 256;
        if (c < hd) {
          float o[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            float t = x[i][j] * rstd;
            if (p.use_norm) t = Elem<T>::rnd(t * wv[i][j]);     // the normalised tensor has type T in the reference
            o[j] = t * gate;
          }
          Elem<T>::store4(dst + c, o[0], o[1], o[2], o[3]);
        }
      }
    } else {
      // n = x rstd; t = n w; y = t g.   dt = dy g; dg = <dy, t>; dn = dt w; dw += dt n; dx = rstd (dn - n mean(dn n))
      const T* dyp = reinterpret_cast<const T*>(p.dy) + yi;
      float dn[LAYER_VEC_MAX][4];
      float dg = 0.f, dnn = 0.f;
#pragma unroll
      for (int i = 0; i < LAYER_VEC_MAX; ++i) {
        const int c = lane * 4 + i * 256;
        if (c < hd) {
          float dyv[4];
          Elem<T>::load4(dyp + c, dyv);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float n = x[i][j] * rstd;
            const float t = p.use_norm ? n * wv[i][j] : n;
            dg += dyv[j] * t;
            const float dt = dyv[j] * gate;
            if (p.use_norm) {
              dwacc[i][j] += dt * n;
              dn[i][j] = dt * wv[i][j];
              dnn += dn[i][j] * n;
            } else {
              dn[i][j] = dt;
            }
          }
        }
      }
      dg = wave_sum(dg);
      if (p.use_norm) dnn = wave_sum(dnn) / (float)hd;
      if (p.gate_raw && lane == 0)
        Elem<T>::store(reinterpret_cast<T*>(p.dgate_raw) + bl * p.g.H + h, dg * silu_grad_f(graw));
      T* dx = reinterpret_cast<T*>(p.d_o) + oi;
#pragma unroll
      for (int i = 0; i < LAYER_VEC_MAX; ++i) {
        const int c = lane * 4 + i * 256;
        if (c < hd) {
          float o[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = p.use_norm ? rstd * (dn[i][j] - x[i][j] * rstd * dnn) : dn[i][j];
          Elem<T>::store4(dx + c, o[0], o[1], o[2], o[3]);
        }
      }
    }
  }
  if (BWD && p.dw_part) {
    float* dst = p.dw_part + ((size_t)blockIdx.x * 4 + wave) * hd;
#pragma unroll
    for (int i = 0; i < LAYER_VEC_MAX; ++i) {
      const int c = lane * 4 + i * 256;
      if (c < hd) *reinterpret_cast<float4*>(dst + c) = make_float4(dwacc[i][0], dwacc[i][1], dwacc[i][2], dwacc[i][3]);
    }
  }
}

}  // namespace lact
