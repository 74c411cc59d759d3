// Fast-weight state kernels: everything that is O(d*dh) per head and update step --
// momentum, Frobenius normalisation for Newton-Schulz, weight update with per-row L2 renorm,
// and their backward passes.  All reductions are deterministic (fixed partial slots, fixed order).
//
// Matrices are packed as [3][b][rows*cols] with index 0: w0 [dh,d], 1: w1 [d,dh], 2: w2 [dh,d].
// Newton-Schulz works on [r,c] = [min(d,dh), max(d,dh)]; a matrix with rows > cols is held
// transposed there (ttt_operation.py:46-47,64-65).
#pragma once
#include "common.h"

namespace lact {

struct MatGeom {
  int d, dh, nb;          // feature dim, hidden dim, batch*heads
  long long elems;        // d*dh
  int stacked;            // Newton-Schulz runs on cat(dw0, dw2) [2dh, d] and on dw1 (fused-kernel variant) instead of three matrices
  __host__ __device__ int rows(int j) const { return j == 1 ? d : dh; }
  __host__ __device__ int cols(int j) const { return j == 1 ? dh : d; }
  __host__ __device__ bool tall(int j) const { return rows(j) > cols(j); }
  __host__ __device__ int maxrows() const { return d > dh ? d : dh; }
  // ---- Newton-Schulz matrices.  They live in buffers of 3*nb*elems elements in "Newton-Schulz orientation"
  // [r, c] = [min, max] (a matrix with more rows than columns is held transposed).  Unstacked: matrix z of the
  // packed order at z*elems.  Stacked: nb matrices of 2*elems (w0 rows on top of w2 rows), then nb of elems (w1).
  __host__ __device__ int ns_count() const { return stacked ? 2 * nb : 3 * nb; }
  __host__ __device__ long long ns_elems(int m) const { return stacked && m < nb ? 2 * elems : elems; }
  __host__ __device__ long long ns_base(int m) const { return stacked ? (m < nb ? m * 2 * elems : 2 * nb * elems + (m - nb) * elems) : m * elems; }
  // Newton-Schulz matrix of packed matrix z = j*nb + ib
  __host__ __device__ int ns_of(int z) const { return stacked ? (z / nb == 1 ? z : z % nb) : z; }
  // packed matrices that make up Newton-Schulz matrix m: first and (stacked pair only) second
  __host__ __device__ int ns_part0(int m) const { return m; }
  __host__ __device__ int ns_part1(int m) const { return stacked && m < nb ? 2 * nb + m : -1; }
  // rows of the matrix the orthogonalisation sees for kind j, and whether it is held transposed
  __host__ __device__ int ns_rows(int j) const { return stacked && j != 1 ? 2 * dh : rows(j); }
  __host__ __device__ bool ns_tall(int j) const { return ns_rows(j) > cols(j); }
  // offset, inside its Newton-Schulz matrix, of element e = i*cols + k of packed matrix kind j
  __host__ __device__ long long xidx(int j, long long e) const {
    const int c = cols(j), nr = ns_rows(j);
    const long long i = e / c + (stacked && j == 2 ? dh : 0), k = e % c;
    return ns_tall(j) ? k * nr + i : i * c + k;
  }
  // four consecutive e map to four consecutive offsets
  __host__ __device__ bool x_contiguous(int j) const { return !ns_tall(j); }
  // offset of packed matrix z in the buffer that holds the orthogonalised update in original orientation
  // (stacked: cat(U0, U2) per head, then U1)
  __host__ __device__ long long u_off(int z) const {
    if (!stacked) return z * elems;
    const int j = z / nb, ib = z % nb;
    return j == 0 ? ib * 2 * elems : (j == 2 ? (ib * 2 + 1) * elems : (2 * nb + ib) * elems);
  }
};

// All kernels below move 16 bytes per lane wherever an array is walked in its own order (d and dh are
// multiples of 8, so rows and matrices are multiples of 4 elements); only a matrix that Newton-Schulz holds
// transposed is addressed element by element.  They are bandwidth-bound: what matters is bytes in flight.

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ void st4(float* p, const float4& v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ float4 f4(float a, float b, float c, float d) { return make_float4(a, b, c, d); }
__device__ __forceinline__ float dot4(const float4& a, const float4& b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

// Flat walk of one matrix by the blocks (blockIdx.x) of a (chunks, 3b) grid: [e0, e1), multiples of 4.
struct FlatRange {
  long long e0, e1;
  __device__ __forceinline__ FlatRange(long long elems) {
    const long long per = ((elems / 4 + gridDim.x - 1) / gridDim.x) * 4;
    e0 = blockIdx.x * per;
    e1 = min(e0 + per, elems);
  }
};

// ---- init: row norms of the initial weights, fp32 state copy, compute-type copy -----------------
struct InitParams {
  MatGeom g;
  const float* w[3];      // [b, rows, cols] each
  float* n0;              // [3b][maxrows]
  float* wf;              // [3b][elems]
  void* wc;               // [3b][elems] compute type, or null when the compute type is fp32
};
template <typename T>
__global__ void k_init_state(const InitParams p) {
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= p.g.rows(j)) return;
  const int cols = p.g.cols(j);
  const float* src = p.w[j] + (size_t)ib * p.g.elems + (size_t)row * cols;
  const size_t o = (size_t)z * p.g.elems + (size_t)row * cols;
  float ss = 0.f;
  for (int c = lane * 4; c < cols; c += 256) {
    const float4 v = ld4(src + c);
    ss += dot4(v, v);
    st4(p.wf + o + c, v);
    if (p.wc) Elem<T>::store4(reinterpret_cast<T*>(p.wc) + o + c, v.x, v.y, v.z, v.w);
  }
  ss = wave_sum(ss);
  if (lane == 0) p.n0[(size_t)z * p.g.maxrows() + row] = sqrtf(ss);
}

// ---- mean of the per-token momentum over one chunk (ttt_operation.py:171-172) --------------------
// One launch for the chunks of up to 256 updates: grid (batch, chunks), mbar [chunks][batch].
struct MomentumMeanRanges {
  int start[256], len[256];
};
__global__ void k_momentum_mean(const float* mom, long long bs, const MomentumMeanRanges r, float* mbar) {
  __shared__ float red[16];
  const int start = r.start[blockIdx.y], len = r.len[blockIdx.y];
  const float* m = mom + blockIdx.x * bs + start;
  float s = 0.f;
  for (int t = threadIdx.x; t < len; t += blockDim.x) s += m[t];
  s = block_sum(s, red);
  if (threadIdx.x == 0) mbar[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = s / (float)len;
}

// ---- reduce split partials, add momentum, emit the bf16 Newton-Schulz input ---------------------
struct MomentumPrepParams {
  MatGeom g;
  const float* partial; int nsplit;   // [nsplit][3b][elems]
  const float* m_prev;                // [3b][elems] or null (no momentum / first update uses zeros)
  const float* mbar;                  // [b] or null
  float* d_out;                       // [3b][elems]  dw (+ momentum): new momentum state, pre-Muon gradient (null: nothing reads it)
  float* m_ext[3];                    // caller's momentum outputs [b][elems] (same values as d_out), each nullable
  void* g16;                          // [3b][elems]  d_out cast to the Newton-Schulz type, in its orientation, or null
  float* ss_part;                     // [3b][gridDim.x]
  int round_partial_bf16;             // the reduction GEMM's result is a bf16 tensor in the reference
  ClearWords clear;
};
template <typename TN>
__global__ void k_momentum_prep(const MomentumPrepParams p) {
  __shared__ float red[16];
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  clear_words(p.clear, blockIdx.x == 0 && blockIdx.y == 0);
  const FlatRange R(p.g.elems);
  const float mb = (p.m_prev && p.mbar) ? p.mbar[ib] : 0.f;
  const size_t zo = (size_t)z * p.g.elems, stride = (size_t)3 * p.g.nb * p.g.elems;
  float* ext = p.m_ext[j] ? p.m_ext[j] + (size_t)ib * p.g.elems : nullptr;
  const bool contiguous = p.g.x_contiguous(j);
  const size_t xo = p.g.ns_base(p.g.ns_of(z));
  float ss = 0.f;
  for (long long e = R.e0 + threadIdx.x * 4; e < R.e1; e += blockDim.x * 4) {
    float4 v = ld4(p.partial + zo + e);
    for (int s = 1; s < p.nsplit; ++s) {
      const float4 t = ld4(p.partial + s * stride + zo + e);
      v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
    }
    if (p.round_partial_bf16) v = f4(round_bf16(v.x), round_bf16(v.y), round_bf16(v.z), round_bf16(v.w));
    if (p.m_prev) {
      const float4 m = ld4(p.m_prev + zo + e);
      // product and sum rounded separately, as the reference's two tensor operations are (ttt_operation.py:174-176)
      v.x = __fadd_rn(v.x, __fmul_rn(m.x, mb)); v.y = __fadd_rn(v.y, __fmul_rn(m.y, mb));
      v.z = __fadd_rn(v.z, __fmul_rn(m.z, mb)); v.w = __fadd_rn(v.w, __fmul_rn(m.w, mb));
    }
    if (p.d_out) st4(p.d_out + zo + e, v);
    if (ext) st4(ext + e, v);
    if (p.g16) {
      const float4 f = f4(Elem<TN>::rnd(v.x), Elem<TN>::rnd(v.y), Elem<TN>::rnd(v.z), Elem<TN>::rnd(v.w));
      TN* g = reinterpret_cast<TN*>(p.g16) + xo;
      if (contiguous) {
        Elem<TN>::store4(g + p.g.xidx(j, e), f.x, f.y, f.z, f.w);
      } else {
        Elem<TN>::store(g + p.g.xidx(j, e), f.x); Elem<TN>::store(g + p.g.xidx(j, e + 1), f.y);
        Elem<TN>::store(g + p.g.xidx(j, e + 2), f.z); Elem<TN>::store(g + p.g.xidx(j, e + 3), f.w);
      }
      ss += dot4(f, f);
    }
  }
  if (p.g16) {
    ss = block_sum(ss, red);
    if (threadIdx.x == 0) p.ss_part[(size_t)z * gridDim.x + blockIdx.x] = ss;
  }
}

// ---- X0 = G / (||G||_F + 1e-7)  (ttt_operation.py:49) -------------------------------------------
struct NsScaleParams {
  MatGeom g;
  const void* g16; const float* ss_part; int nparts;
  float* norms;          // [3b]
  float* xf; void* xb;   // [3b][elems], Newton-Schulz orientation (fp32 iterate, copy in the Newton-Schulz type)
  float* u;              // [3b][elems] original orientation, or null (only when zero iterations follow)
  int plain_bf16;        // reference without autocast: norm and quotient are bf16 tensors
  ClearWords clear;
};
// Grid (chunks, Newton-Schulz matrices).  ss_part is indexed by packed matrix.
template <typename TN>
__global__ void k_ns_scale(const NsScaleParams p) {
  const int m = blockIdx.y;
  clear_words(p.clear, blockIdx.x == 0 && blockIdx.y == 0);
  float ss = 0.f;
  for (int i = 0; i < p.nparts; ++i) ss += p.ss_part[(size_t)p.g.ns_part0(m) * p.nparts + i];
  if (p.g.ns_part1(m) >= 0)
    for (int i = 0; i < p.nparts; ++i) ss += p.ss_part[(size_t)p.g.ns_part1(m) * p.nparts + i];
  float n = sqrtf(ss);
  if (p.plain_bf16) n = round_bf16(n);
  if (blockIdx.x == 0 && threadIdx.x == 0) p.norms[m] = n;
  float den = n + 1e-7f;
  if (p.plain_bf16) den = round_bf16(den);
  const FlatRange R(p.g.ns_elems(m));
  const size_t zo = p.g.ns_base(m);
  // `u` (only when zero iterations follow; never stacked): original orientation of matrix m = packed z
  const int j = m / p.g.nb;
  const bool tall = p.g.tall(j);
  for (long long x = R.e0 + threadIdx.x * 4; x < R.e1; x += blockDim.x * 4) {
    float v[4];
    Elem<TN>::load4(reinterpret_cast<const TN*>(p.g16) + zo + x, v);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = __fdiv_rn(v[i], den);   // the quotient itself (ttt_operation.py:49), not a product with 1 / den
      if (p.plain_bf16) v[i] = round_bf16(v[i]);
    }
    st4(p.xf + zo + x, f4(v[0], v[1], v[2], v[3]));
    Elem<TN>::store4(reinterpret_cast<TN*>(p.xb) + zo + x, v[0], v[1], v[2], v[3]);
    if (p.u) {
      if (!tall) {
        st4(p.u + zo + x, f4(v[0], v[1], v[2], v[3]));
      } else {   // x = k*rows + i  ->  e = i*cols + k
        const int rows = p.g.rows(j), cols = p.g.cols(j);
#pragma unroll
        for (int i = 0; i < 4; ++i) p.u[zo + (size_t)((x + i) % rows) * cols + (x + i) / rows] = v[i];
      }
    }
  }
}

// ---- w_hat = cw*base + U + cr*D ;  w = w_hat / (||w_hat||_row + 1e-5) * n0  (ttt_operation.py:193-200)
struct RenormParams {
  MatGeom g;
  const float* base; float cw;     // previous weights (post-norm) or accumulator (pre-norm)
  const float* u;                  // orthogonalised (or raw) gradient, original orientation
  const float* raw; float cr;      // raw gradient added on top (bidirectional layer), or null
  const float* n0;
  int weight_norm;
  int u_stacked;                   // `u` is laid out per Newton-Schulz matrix (MatGeom::u_off), not packed
  int eps_in_sqrt;                 // y = w_hat / sqrt(|w_hat|^2 + eps) * n0 (fused-kernel variant) instead of / (|w_hat| + eps)
  float* main_out;                 // un-normalised accumulator (pre-norm) or null
  float* wf_out; void* wc_out;     // new weights: fp32 state and compute-type copy (each may be null)
  float* w_ext[3];                 // caller's weight outputs [b][elems] (same values as wf_out), each nullable
  const unsigned* poison;          // nonzero word: an earlier kernel of this step failed (barrier timeout) -> results become NaN
  // backward only
  const float* gy;                 // gradient w.r.t. the new weights, or null (= zero)
  const float* gy2;                // second addend of the same gradient (the apply steps' share), or null
  const float* carry_in;           // gradient arriving at the accumulator from later steps (pre-norm) or null
  float* gw_hat;                   // gradient w.r.t. w_hat, original orientation
  float* gn0;                      // [3b][maxrows], accumulated (written when gn0_init: first use in a backward pass)
  int gn0_init;
  ClearWords clear;
  float* gxf; void* gxb;           // the same gradient in Newton-Schulz orientation (fp32 + Newton-Schulz type) or null
};
// off: offset in the packed arrays; uo: offset of the same element in `u`
__device__ __forceinline__ float4 renorm_w_hat4(const RenormParams& p, size_t off, size_t uo) {
  float4 v = ld4(p.u + uo);
  if (p.cw != 0.f) {
    const float4 b = ld4(p.base + off);
    v.x += p.cw * b.x; v.y += p.cw * b.y; v.z += p.cw * b.z; v.w += p.cw * b.w;
  }
  if (p.raw) {
    const float4 r = ld4(p.raw + off);
    v.x += p.cr * r.x; v.y += p.cr * r.y; v.z += p.cr * r.z; v.w += p.cr * r.w;
  }
  return v;
}
__device__ __forceinline__ float4 renorm_gy4(const RenormParams& p, size_t off) {
  float4 g = p.gy ? ld4(p.gy + off) : f4(0.f, 0.f, 0.f, 0.f);
  if (p.gy2) {
    const float4 t = ld4(p.gy2 + off);
    g.x += t.x; g.y += t.y; g.z += t.z; g.w += t.w;
  }
  return g;
}
constexpr int ROW_VEC_MAX = 4;   // a lane keeps up to 4 x 4 elements of its row in registers (rows up to 1024 columns)
template <typename T>
__global__ void k_update_renorm(const RenormParams p) {
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= p.g.rows(j)) return;
  const int cols = p.g.cols(j);
  const size_t o = (size_t)z * p.g.elems + (size_t)row * cols;
  const size_t uo = (p.u_stacked ? (size_t)p.g.u_off(z) : (size_t)z * p.g.elems) + (size_t)row * cols;
  float* ext = p.w_ext[j] ? p.w_ext[j] + (size_t)ib * p.g.elems + (size_t)row * cols : nullptr;
  const bool keep = cols <= 256 * ROW_VEC_MAX;
  float4 vv[ROW_VEC_MAX];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < ROW_VEC_MAX; ++i) {
    const int c = lane * 4 + i * 256;
    if (c < cols) {
      vv[i] = renorm_w_hat4(p, o + c, uo + c);
      ss += dot4(vv[i], vv[i]);
    }
  }
  for (int c = lane * 4 + ROW_VEC_MAX * 256; c < cols; c += 256) {
    const float4 v = renorm_w_hat4(p, o + c, uo + c);
    ss += dot4(v, v);
  }
  ss = wave_sum(ss);
  float den = p.eps_in_sqrt ? sqrtf(ss + 1e-5f) : sqrtf(ss) + 1e-5f;
  if (p.poison && *p.poison) den = __uint_as_float(0x7fc00000u);
  const float n0 = p.weight_norm ? p.n0[(size_t)z * p.g.maxrows() + row] : 1.f;
  auto emit = [&](int c, const float4& v) {
    if (p.main_out) st4(p.main_out + o + c, v);
    // same operation order as the reference: (w / (norm + eps)) * w_norm
    const float4 y = p.weight_norm ? f4((v.x / den) * n0, (v.y / den) * n0, (v.z / den) * n0, (v.w / den) * n0)
                                   : f4(v.x + 0.f * den, v.y + 0.f * den, v.z + 0.f * den, v.w + 0.f * den);
    if (p.wf_out) st4(p.wf_out + o + c, y);
    if (ext) st4(ext + c, y);
    if (p.wc_out) Elem<T>::store4(reinterpret_cast<T*>(p.wc_out) + o + c, y.x, y.y, y.z, y.w);
  };
#pragma unroll
  for (int i = 0; i < ROW_VEC_MAX; ++i) {
    const int c = lane * 4 + i * 256;
    if (c < cols) emit(c, vv[i]);
  }
  if (!keep)
    for (int c = lane * 4 + ROW_VEC_MAX * 256; c < cols; c += 256) emit(c, renorm_w_hat4(p, o + c, uo + c));
}

// backward of the line above.  y = w_hat*n0/(r+eps), r = ||w_hat||:
//   g_w_hat = gy*n0/(r+eps) - w_hat * <gy,w_hat> * n0 / (r (r+eps)^2),   g_n0 = <gy,w_hat>/(r+eps)
template <typename TN>
__global__ void k_renorm_bwd(const RenormParams p) {
  const int z = blockIdx.y, j = z / p.g.nb;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  clear_words(p.clear, blockIdx.x == 0 && blockIdx.y == 0);
  if (row >= p.g.rows(j)) return;
  const int cols = p.g.cols(j);
  const size_t o = (size_t)z * p.g.elems + (size_t)row * cols;
  const size_t uo = (p.u_stacked ? (size_t)p.g.u_off(z) : (size_t)z * p.g.elems) + (size_t)row * cols;
  const size_t xo = p.g.ns_base(p.g.ns_of(z));
  const bool contiguous = p.g.x_contiguous(j);
  float c0 = 1.f, c1 = 0.f;
  float* gn0 = p.gn0 + (size_t)z * p.g.maxrows() + row;
  if (!p.weight_norm && p.gn0_init && lane == 0) *gn0 = 0.f;
  // the first 1024 columns of a row stay in registers between the two passes (as in k_update_renorm)
  float4 wv[ROW_VEC_MAX], gk[ROW_VEC_MAX];
  if (p.weight_norm) {
    float ss = 0.f, dot = 0.f;
#pragma unroll
    for (int i = 0; i < ROW_VEC_MAX; ++i) {
      const int c = lane * 4 + i * 256;
      if (c < cols) {
        wv[i] = renorm_w_hat4(p, o + c, uo + c);
        gk[i] = renorm_gy4(p, o + c);
        ss += dot4(wv[i], wv[i]);
        if (p.gy || p.gy2) dot += dot4(wv[i], gk[i]);
      }
    }
    for (int c = lane * 4 + ROW_VEC_MAX * 256; c < cols; c += 256) {
      const float4 v = renorm_w_hat4(p, o + c, uo + c);
      ss += dot4(v, v);
      if (p.gy || p.gy2) dot += dot4(v, renorm_gy4(p, o + c));
    }
    ss = wave_sum(ss);
    dot = wave_sum(dot);
    const float n0 = p.n0[(size_t)z * p.g.maxrows() + row];
    if (p.eps_in_sqrt) {   // den = sqrt(r^2 + eps):  d den / d w = w / den
      const float den = sqrtf(ss + 1e-5f);
      c0 = n0 / den;
      c1 = dot * n0 / (den * den * den);
      if (lane == 0) *gn0 = (p.gn0_init ? 0.f : *gn0) + dot / den;
    } else {               // den = r + eps:  d den / d w = w / r
      const float r = sqrtf(ss);
      c0 = n0 / (r + 1e-5f);
      c1 = r > 0.f ? dot * n0 / (r * (r + 1e-5f) * (r + 1e-5f)) : 0.f;
      if (lane == 0) *gn0 = (p.gn0_init ? 0.f : *gn0) + dot / (r + 1e-5f);
    }
  }
  auto emit = [&](int c, float4 gv, const float4& w) {
    gv = f4(gv.x * c0, gv.y * c0, gv.z * c0, gv.w * c0);
    if (p.weight_norm) {
      gv.x -= w.x * c1; gv.y -= w.y * c1; gv.z -= w.z * c1; gv.w -= w.w * c1;
    }
    if (p.carry_in) {
      const float4 ci = ld4(p.carry_in + o + c);
      gv.x += ci.x; gv.y += ci.y; gv.z += ci.z; gv.w += ci.w;
    }
    st4(p.gw_hat + o + c, gv);
    if (p.gxf) {   // the same gradient where Newton-Schulz holds this matrix
      const long long e = (long long)row * cols + c;
      if (contiguous) {
        const size_t x = xo + p.g.xidx(j, e);
        st4(p.gxf + x, gv);
        Elem<TN>::store4(reinterpret_cast<TN*>(p.gxb) + x, gv.x, gv.y, gv.z, gv.w);
      } else {
        const float g[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const size_t x = xo + p.g.xidx(j, e + i);
          p.gxf[x] = g[i];
          Elem<TN>::store(reinterpret_cast<TN*>(p.gxb) + x, g[i]);
        }
      }
    }
  };
  const float4 zero4 = f4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int i = 0; i < ROW_VEC_MAX; ++i) {
    const int c = lane * 4 + i * 256;
    if (c < cols) {
      if (p.weight_norm) emit(c, gk[i], wv[i]);
      else emit(c, renorm_gy4(p, o + c), zero4);
    }
  }
  for (int c = lane * 4 + ROW_VEC_MAX * 256; c < cols; c += 256)
    emit(c, renorm_gy4(p, o + c), p.weight_norm ? renorm_w_hat4(p, o + c, uo + c) : zero4);
}

// A gradient given in the original orientation of its matrices, copied to where Newton-Schulz holds them (fp32 and
// Newton-Schulz type).  Grid (chunks, matrices).
template <typename TN>
__global__ void k_to_ns_orientation(const MatGeom g, const float* in, float* xf, void* xb) {
  const int z = blockIdx.y, j = z / g.nb;
  const FlatRange R(g.elems);
  const size_t zo = (size_t)z * g.elems, xo = g.ns_base(g.ns_of(z));
  const bool contiguous = g.x_contiguous(j);
  for (long long e = R.e0 + threadIdx.x * 4; e < R.e1; e += blockDim.x * 4) {
    const float4 v = ld4(in + zo + e);
    if (contiguous) {
      const size_t x = xo + g.xidx(j, e);
      st4(xf + x, v);
      Elem<TN>::store4(reinterpret_cast<TN*>(xb) + x, v.x, v.y, v.z, v.w);
    } else {
      const float a[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const size_t x = xo + g.xidx(j, e + i);
        xf[x] = a[i];
        Elem<TN>::store(reinterpret_cast<TN*>(xb) + x, a[i]);
      }
    }
  }
}

// ---- backward of the Frobenius normalisation, the momentum recurrence and the raw-gradient add --
struct NsDotParams {
  MatGeom g;
  const float* gx0; const void* g16; float* dot_part;
};
// Grid (chunks, Newton-Schulz matrices): <gradient at X0, Newton-Schulz input> per matrix.
template <typename TN>
__global__ void k_ns_bwd_dot(const NsDotParams p) {
  __shared__ float red[16];
  const int m = blockIdx.y;
  const FlatRange R(p.g.ns_elems(m));
  const size_t zo = p.g.ns_base(m);
  float s = 0.f;
  for (long long e = R.e0 + threadIdx.x * 4; e < R.e1; e += blockDim.x * 4) {
    float g[4];
    Elem<TN>::load4(reinterpret_cast<const TN*>(p.g16) + zo + e, g);
    s += dot4(ld4(p.gx0 + zo + e), f4(g[0], g[1], g[2], g[3]));
  }
  s = block_sum(s, red);
  if (threadIdx.x == 0) p.dot_part[(size_t)m * gridDim.x + blockIdx.x] = s;
}

// Gradient w.r.t. the Newton-Schulz input G16 (type TN) of X0 = G16 / (|G16| + 1e-7), from the gradient gx of X0:
// gx * c0 through the quotient, -g16 * c1 through the norm (c0 = 1 / (n + eps), c1 = <gx, G16> / (n (n + eps)^2)).
template <typename TN>
__device__ __forceinline__ float ns_input_grad(float gx, float g16, float c0, float c1) {
  return Elem<TN>::rnd(Elem<TN>::rnd(gx * c0) - Elem<TN>::rnd(g16 * c1));
}

struct GradPrepParams {
  MatGeom g;
  int muon;
  const float* gx0; const void* g16; const float* norms; const float* dot_part; int nparts;
  const float* gw_hat; float cr;     // added when the raw gradient also enters w_hat
  float* gm_carry; int carry_valid;  // gradient w.r.t. the momentum state after this update (in/out)
  int carry_write;                   // an earlier update exists: hand it gm_carry = g * mbar
  const float* m_prev; const float* mbar;   // null without momentum
  void* gc;                          // [3b][elems] compute-type copy of d loss / d dw  (GEMM operand)
  float* mdot_part;                  // [3b][gridDim.x] partial <g, m_prev>
  const unsigned* poison;            // nonzero word: an earlier kernel of this step failed (barrier timeout) -> results become NaN
};
template <typename T, typename TN>
__global__ void k_grad_prep(const GradPrepParams p) {
  __shared__ float red[16];
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  float c0 = 1.f, c1 = 0.f;
  if (p.muon) {
    const int m = p.g.ns_of(z);
    float dot = 0.f;
    for (int i = 0; i < p.nparts; ++i) dot += p.dot_part[(size_t)m * p.nparts + i];
    const float n = p.norms[m];
    c0 = 1.f / (n + 1e-7f);
    c1 = n > 0.f ? dot / (n * (n + 1e-7f) * (n + 1e-7f)) : 0.f;
    if (p.poison && *p.poison) c0 = __uint_as_float(0x7fc00000u);
  }
  const float mb = p.mbar ? p.mbar[ib] : 0.f;
  const FlatRange R(p.g.elems);
  const size_t zo = (size_t)z * p.g.elems;
  const size_t xo = p.g.ns_base(p.g.ns_of(z));
  const bool contiguous = p.g.x_contiguous(j);
  float md = 0.f;
  for (long long e = R.e0 + threadIdx.x * 4; e < R.e1; e += blockDim.x * 4) {
    const size_t o = zo + e;
    float4 gv;
    if (p.muon) {
      float4 gx;
      float g[4];
      if (contiguous) {
        const size_t x = xo + p.g.xidx(j, e);
        gx = ld4(p.gx0 + x);
        Elem<TN>::load4(reinterpret_cast<const TN*>(p.g16) + x, g);
      } else {
        float t[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const size_t x = xo + p.g.xidx(j, e + i);
          t[i] = p.gx0[x];
          g[i] = Elem<TN>::load(reinterpret_cast<const TN*>(p.g16) + x);
        }
        gx = f4(t[0], t[1], t[2], t[3]);
      }
      // the gradient that leaves Newton-Schulz through its input cast (G.bfloat16(), ttt_operation.py:45) has that type
      // (two gradients arrive there, through the quotient and through the norm, :49; each is a tensor of that type, and so is their sum)
      gv = f4(ns_input_grad<TN>(gx.x, g[0], c0, c1), ns_input_grad<TN>(gx.y, g[1], c0, c1), ns_input_grad<TN>(gx.z, g[2], c0, c1),
              ns_input_grad<TN>(gx.w, g[3], c0, c1));
      if (p.cr != 0.f) {
        const float4 w = ld4(p.gw_hat + o);
        gv.x += p.cr * w.x; gv.y += p.cr * w.y; gv.z += p.cr * w.z; gv.w += p.cr * w.w;
      }
    } else {
      gv = ld4(p.gw_hat + o);
    }
    if (p.gm_carry) {
      if (p.carry_valid) {
        const float4 cv = ld4(p.gm_carry + o);
        gv.x += cv.x; gv.y += cv.y; gv.z += cv.z; gv.w += cv.w;
      }
      if (p.carry_write) st4(p.gm_carry + o, f4(gv.x * mb, gv.y * mb, gv.z * mb, gv.w * mb));   // d/d M_prev of  dw + M_prev * mbar
      if (p.m_prev) md += dot4(gv, ld4(p.m_prev + o));
    }
    Elem<T>::store4(reinterpret_cast<T*>(p.gc) + o, gv.x, gv.y, gv.z, gv.w);
  }
  if (p.gm_carry && p.m_prev) {
    md = block_sum(md, red);
    if (threadIdx.x == 0) p.mdot_part[(size_t)z * gridDim.x + blockIdx.x] = md;
  }
}

// d loss / d momentum[t] = <g, M_prev> / chunk_len for every token of the chunk (mean, :172).  Grid (batch, updates):
// update i of the launch has its partial dot products at mdot_part + i * slot_stride and the token range r[i]; the
// ranges of one launch do not overlap (each row is written by one block).
__global__ void k_momentum_grad(const float* mdot_part, long long slot_stride, int nparts, int nb, float* dmom, long long bs,
                                const MomentumMeanRanges r, int accumulate) {
  const int ib = blockIdx.x;
  const float* part = mdot_part + blockIdx.y * slot_stride;
  const int start = r.start[blockIdx.y], len = r.len[blockIdx.y];
  float s = 0.f;
  for (int j = 0; j < 3; ++j)
    for (int i = 0; i < nparts; ++i) s += part[(size_t)(j * nb + ib) * nparts + i];
  s /= (float)len;
  for (int t = threadIdx.x; t < len; t += blockDim.x) {
    float* dst = dmom + ib * bs + start + t;
    *dst = accumulate ? *dst + s : s;
  }
}

// out = coeff*in_add + sum of split partials; 4 elements per thread (total is a multiple of 4)
__global__ void k_reduce_partials(float* out, const float* in_add, float coeff, const float* partial, int nsplit, long long total) {
  const long long e = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (e >= total) return;
  float4 v = f4(0.f, 0.f, 0.f, 0.f);
  if (in_add) {
    const float4 a = ld4(in_add + e);
    v = f4(coeff * a.x, coeff * a.y, coeff * a.z, coeff * a.w);
  }
  for (int s = 0; s < nsplit; ++s) {
    const float4 t = ld4(partial + (size_t)s * total + e);
    v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
  }
  st4(out + e, v);
}

// dlr_j[ib, start + t] = (or +=, on rows an earlier step of this call wrote) sum over slots of the row partials.
// Grid (ceil(longest chunk / 256), batch, 3 * updates): update i of the launch has its partials at
// lrpart + i * upd_stride and the token range r[i]; the ranges of one launch do not overlap.
__global__ void k_lr_reduce(const float* lrpart, long long upd_stride, long long mat_stride, long long slot_stride, int nslots, int Tcap,
                            float* dlr0, float* dlr1, float* dlr2, long long bs, const MomentumMeanRanges r, int accumulate) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x, ib = blockIdx.y, j = blockIdx.z % 3, i = blockIdx.z / 3;
  const int start = r.start[i], len = r.len[i];
  if (t >= len) return;
  const float* part = lrpart + i * upd_stride;
  float s = 0.f;
  for (int k = 0; k < nslots; ++k) s += part[j * mat_stride + k * slot_stride + (size_t)ib * Tcap + t];
  float* dst = j == 0 ? dlr0 : (j == 1 ? dlr1 : dlr2);
  dst += ib * bs + start + t;
  *dst = accumulate ? *dst + s : s;
}

// final weight gradients: state gradient (+ accumulator carry) + the path through the initial row norms
struct FinishParams {
  MatGeom g;
  const float* gw; const float* gw2; const float* carry; const float* gn0; const float* n0; const float* w_init;   // gw, gw2: addends, nullable
  int through_norms;
  float* out[3];
};
__global__ void k_finish_weight_grads(const FinishParams p) {
  // flat over a matrix, 4 consecutive elements per thread (a row holds a multiple of 4): every lane works
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  const long long e = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (e >= p.g.elems) return;
  const int cols = p.g.cols(j), row = (int)(e / cols);
  const size_t o = (size_t)z * p.g.elems + e;
  float4 v = p.gw ? ld4(p.gw + o) : f4(0.f, 0.f, 0.f, 0.f);
  if (p.gw2) {
    const float4 t = ld4(p.gw2 + o);
    v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
  }
  if (p.carry) {
    const float4 t = ld4(p.carry + o);
    v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
  }
  if (p.through_norms) {
    const float n = p.n0[(size_t)z * p.g.maxrows() + row];
    const float c = n > 0.f ? p.gn0[(size_t)z * p.g.maxrows() + row] / n : 0.f;
    const float4 w = ld4(p.w_init + o);
    v.x += c * w.x; v.y += c * w.y; v.z += c * w.z; v.w += c * w.w;
  }
  st4(p.out[j] + (size_t)ib * p.g.elems + e, v);
}

// [3b][elems] <-> the three caller tensors, 4 elements per thread
__global__ void k_unpack3(const float* src, long long elems, int nb, float* o0, float* o1, float* o2) {
  const long long e = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int z = blockIdx.y;
  if (e >= elems) return;
  float* dst = (z / nb) == 0 ? o0 : ((z / nb) == 1 ? o1 : o2);
  if (dst) st4(dst + (size_t)(z % nb) * elems + e, ld4(src + (size_t)z * elems + e));
}
__global__ void k_pack3(float* dst, long long elems, int nb, const float* i0, const float* i1, const float* i2) {
  const long long e = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int z = blockIdx.y;
  if (e >= elems) return;
  const float* src = (z / nb) == 0 ? i0 : ((z / nb) == 1 ? i1 : i2);
  st4(dst + (size_t)z * elems + e, src ? ld4(src + (size_t)(z % nb) * elems + e) : f4(0.f, 0.f, 0.f, 0.f));
}

// Zero up to 16 strided byte ranges in one launch: segment i covers, for every batch ib < nb, the bytes
// [ptr + ib*bs + off, +len); everything a multiple of 4 bytes.  Grid (chunks of 4 KiB, nb, segments).
struct ZeroSegments {
  char* ptr[16];
  long long bs[16], off[16], len[16];
};
__global__ void k_zero_segments(const ZeroSegments z) {
  const int i = blockIdx.z;
  const long long e = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 16;
  if (e >= z.len[i]) return;
  char* dst = z.ptr[i] + blockIdx.y * z.bs[i] + z.off[i] + e;
  if ((reinterpret_cast<uintptr_t>(dst) & 15) == 0 && e + 16 <= z.len[i]) {
    *reinterpret_cast<uint4*>(dst) = make_uint4(0, 0, 0, 0);
  } else {   // lengths are multiples of 4 bytes
    for (int j = 0; j < 16 && e + j < z.len[i]; j += 4) *reinterpret_cast<uint32_t*>(dst + j) = 0u;
  }
}

__global__ void k_fill_f32(float* p, float v, long long n) {
  const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e < n) p[e] = v;
}

}  // namespace lact
