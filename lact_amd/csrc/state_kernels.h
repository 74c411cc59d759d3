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
  __host__ __device__ int rows(int j) const { return j == 1 ? d : dh; }
  __host__ __device__ int cols(int j) const { return j == 1 ? dh : d; }
  __host__ __device__ bool tall(int j) const { return rows(j) > cols(j); }
  __host__ __device__ int maxrows() const { return d > dh ? d : dh; }
  // Newton-Schulz orientation is [r, c] = [min, max]; index of the same element in the [c, r] transpose
  __device__ long long xtidx(long long x) const {
    const int r = d < dh ? d : dh, c = d < dh ? dh : d;
    return (x % c) * r + x / c;
  }
  // index of original element e = i*cols + j inside the Newton-Schulz orientation
  __device__ long long xidx(int j, long long e) const {
    if (!tall(j)) return e;
    const int c = cols(j), r = rows(j);
    const long long i = e / c, k = e % c;
    return k * r + i;
  }
};

// ---- init: row norms of the initial weights, fp32 state copy, compute-type copy -----------------
struct InitParams {
  MatGeom g;
  const float* w[3];      // [b, rows, cols] each
  float* n0;              // [3b][maxrows]
  float* wf;              // [3b][elems]
  void* wc;               // [3b][elems] compute type, or null when the compute type is fp32
  uint16_t* wct;          // [3b][elems] bf16, each matrix transposed ([cols][rows]), or null
};
template <typename T>
__global__ void k_init_state(const InitParams p) {
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= p.g.rows(j)) return;
  const int cols = p.g.cols(j);
  const float* src = p.w[j] + (size_t)ib * p.g.elems + (size_t)row * cols;
  float* dst = p.wf + (size_t)z * p.g.elems + (size_t)row * cols;
  float ss = 0.f;
  for (int c = lane; c < cols; c += 64) {
    const float v = src[c];
    ss += v * v;
    dst[c] = v;
    if (p.wc) Elem<T>::store(reinterpret_cast<T*>(p.wc) + (size_t)z * p.g.elems + (size_t)row * cols + c, v);
    if (p.wct) p.wct[(size_t)z * p.g.elems + (size_t)c * p.g.rows(j) + row] = f32_to_bf16(v);
  }
  ss = wave_sum(ss);
  if (lane == 0) p.n0[(size_t)z * p.g.maxrows() + row] = sqrtf(ss);
}

// ---- mean of the per-token momentum over one chunk (ttt_operation.py:171-172) --------------------
__global__ void k_momentum_mean(const float* mom, long long bs, int start, int len, float* mbar) {
  __shared__ float red[16];
  const float* m = mom + blockIdx.x * bs + start;
  float s = 0.f;
  for (int t = threadIdx.x; t < len; t += blockDim.x) s += m[t];
  s = block_sum(s, red);
  if (threadIdx.x == 0) mbar[blockIdx.x] = s / (float)len;
}

// ---- reduce split partials, add momentum, emit the bf16 Newton-Schulz input ---------------------
struct MomentumPrepParams {
  MatGeom g;
  const float* partial; int nsplit;   // [nsplit][3b][elems]
  const float* m_prev;                // [3b][elems] or null (no momentum / first update uses zeros)
  const float* mbar;                  // [b] or null
  float* d_out;                       // [3b][elems]  dw (+ momentum): new momentum state, pre-Muon gradient
  void* g16;                          // [3b][elems]  d_out cast to the Newton-Schulz type, in its orientation, or null
  float* ss_part;                     // [3b][gridDim.x]
  int round_partial_bf16;             // the reduction GEMM's result is a bf16 tensor in the reference
};
template <typename TN>
__global__ void k_momentum_prep(const MomentumPrepParams p) {
  __shared__ float red[16];
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  const long long per = (p.g.elems + gridDim.x - 1) / gridDim.x;
  const long long e0 = blockIdx.x * per, e1 = min(e0 + per, p.g.elems);
  const float mb = (p.m_prev && p.mbar) ? p.mbar[ib] : 0.f;
  float ss = 0.f;
  for (long long e = e0 + threadIdx.x; e < e1; e += blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < p.nsplit; ++s) v += p.partial[((size_t)s * 3 * p.g.nb + z) * p.g.elems + e];
    if (p.round_partial_bf16) v = round_bf16(v);
    if (p.m_prev) v += p.m_prev[(size_t)z * p.g.elems + e] * mb;
    p.d_out[(size_t)z * p.g.elems + e] = v;
    if (p.g16) {
      const float f = Elem<TN>::rnd(v);
      Elem<TN>::store(reinterpret_cast<TN*>(p.g16) + (size_t)z * p.g.elems + p.g.xidx(j, e), f);
      ss += f * f;
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
  uint16_t* xbt;         // [3b][elems] bf16 copy transposed ([c][r]), or null
  float* u;              // [3b][elems] original orientation, or null (only when zero iterations follow)
  int plain_bf16;        // reference without autocast: norm and quotient are bf16 tensors
};
template <typename TN>
__global__ void k_ns_scale(const NsScaleParams p) {
  const int z = blockIdx.y, j = z / p.g.nb;
  float ss = 0.f;
  for (int i = 0; i < p.nparts; ++i) ss += p.ss_part[(size_t)z * p.nparts + i];
  float n = sqrtf(ss);
  if (p.plain_bf16) n = round_bf16(n);
  if (blockIdx.x == 0 && threadIdx.x == 0) p.norms[z] = n;
  float den = n + 1e-7f;
  if (p.plain_bf16) den = round_bf16(den);
  const float inv = 1.f / den;
  const long long per = (p.g.elems + gridDim.x - 1) / gridDim.x;
  const long long e0 = blockIdx.x * per, e1 = min(e0 + per, p.g.elems);
  for (long long e = e0 + threadIdx.x; e < e1; e += blockDim.x) {
    const long long x = p.g.xidx(j, e);
    float v = Elem<TN>::load(reinterpret_cast<const TN*>(p.g16) + (size_t)z * p.g.elems + x) * inv;
    if (p.plain_bf16) v = round_bf16(v);
    p.xf[(size_t)z * p.g.elems + x] = v;
    Elem<TN>::store(reinterpret_cast<TN*>(p.xb) + (size_t)z * p.g.elems + x, v);
    if (p.xbt) p.xbt[(size_t)z * p.g.elems + p.g.xtidx(x)] = f32_to_bf16(v);
    if (p.u) p.u[(size_t)z * p.g.elems + e] = v;
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
  float* main_out;                 // un-normalised accumulator (pre-norm) or null
  float* wf_out; void* wc_out;     // new weights: fp32 state and compute-type copy (may be null)
  uint16_t* wct_out;               // bf16 transposed copy ([cols][rows]) or null
  uint16_t* gxbt;                  // backward: bf16 transposed copy of the Newton-Schulz-orientation gradient, or null
  // backward only
  const float* gy;                 // gradient w.r.t. the new weights
  const float* carry_in;           // gradient arriving at the accumulator from later steps (pre-norm) or null
  float* gw_hat;                   // gradient w.r.t. w_hat, original orientation
  float* gn0;                      // [3b][maxrows], accumulated
  float* gxf; void* gxb;           // the same gradient in Newton-Schulz orientation (fp32 + Newton-Schulz type) or null
};
__device__ __forceinline__ float renorm_w_hat(const RenormParams& p, size_t off) {
  float v = p.u[off];
  if (p.cw != 0.f) v += p.cw * p.base[off];
  if (p.raw) v += p.cr * p.raw[off];
  return v;
}
template <typename T>
__global__ void k_update_renorm(const RenormParams p) {
  const int z = blockIdx.y, j = z / p.g.nb;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= p.g.rows(j)) return;
  const int cols = p.g.cols(j);
  const size_t o = (size_t)z * p.g.elems + (size_t)row * cols;
  float ss = 0.f;
  for (int c = lane; c < cols; c += 64) {
    const float v = renorm_w_hat(p, o + c);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float den = sqrtf(ss) + 1e-5f;
  const float n0 = p.weight_norm ? p.n0[(size_t)z * p.g.maxrows() + row] : 1.f;
  for (int c = lane; c < cols; c += 64) {
    const float v = renorm_w_hat(p, o + c);
    if (p.main_out) p.main_out[o + c] = v;
    // same operation order as the reference: (w / (norm + eps)) * w_norm
    const float y = p.weight_norm ? (v / den) * n0 : v;
    p.wf_out[o + c] = y;
    if (p.wc_out) Elem<T>::store(reinterpret_cast<T*>(p.wc_out) + o + c, y);
    if (p.wct_out) p.wct_out[(size_t)z * p.g.elems + (size_t)c * p.g.rows(j) + row] = f32_to_bf16(y);
  }
}

// backward of the line above.  y = w_hat*n0/(r+eps), r = ||w_hat||:
//   g_w_hat = gy*n0/(r+eps) - w_hat * <gy,w_hat> * n0 / (r (r+eps)^2),   g_n0 = <gy,w_hat>/(r+eps)
template <typename TN>
__global__ void k_renorm_bwd(const RenormParams p) {
  const int z = blockIdx.y, j = z / p.g.nb;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= p.g.rows(j)) return;
  const int cols = p.g.cols(j);
  const size_t o = (size_t)z * p.g.elems + (size_t)row * cols;
  float c0 = 1.f, c1 = 0.f;
  if (p.weight_norm) {
    float ss = 0.f, dot = 0.f;
    for (int c = lane; c < cols; c += 64) {
      const float v = renorm_w_hat(p, o + c);
      ss += v * v;
      dot += v * p.gy[o + c];
    }
    ss = wave_sum(ss);
    dot = wave_sum(dot);
    const float r = sqrtf(ss), n0 = p.n0[(size_t)z * p.g.maxrows() + row];
    c0 = n0 / (r + 1e-5f);
    c1 = r > 0.f ? dot * n0 / (r * (r + 1e-5f) * (r + 1e-5f)) : 0.f;
    if (lane == 0) p.gn0[(size_t)z * p.g.maxrows() + row] += dot / (r + 1e-5f);
  }
  for (int c = lane; c < cols; c += 64) {
    float gv = p.gy[o + c] * c0;
    if (p.weight_norm) gv -= renorm_w_hat(p, o + c) * c1;
    if (p.carry_in) gv += p.carry_in[o + c];
    p.gw_hat[o + c] = gv;
    if (p.gxf) {
      const size_t x = (size_t)z * p.g.elems + p.g.xidx(j, (long long)row * cols + c);
      p.gxf[x] = gv;
      Elem<TN>::store(reinterpret_cast<TN*>(p.gxb) + x, gv);
      if (p.gxbt) p.gxbt[(size_t)z * p.g.elems + p.g.xtidx(x - (size_t)z * p.g.elems)] = f32_to_bf16(gv);
    }
  }
}

// ---- backward of the Frobenius normalisation, the momentum recurrence and the raw-gradient add --
struct NsDotParams {
  MatGeom g;
  const float* gx0; const void* g16; float* dot_part;
};
template <typename TN>
__global__ void k_ns_bwd_dot(const NsDotParams p) {
  __shared__ float red[16];
  const int z = blockIdx.y;
  const long long per = (p.g.elems + gridDim.x - 1) / gridDim.x;
  const long long e0 = blockIdx.x * per, e1 = min(e0 + per, p.g.elems);
  float s = 0.f;
  for (long long e = e0 + threadIdx.x; e < e1; e += blockDim.x)
    s += p.gx0[(size_t)z * p.g.elems + e] * Elem<TN>::load(reinterpret_cast<const TN*>(p.g16) + (size_t)z * p.g.elems + e);
  s = block_sum(s, red);
  if (threadIdx.x == 0) p.dot_part[(size_t)z * gridDim.x + blockIdx.x] = s;
}

struct GradPrepParams {
  MatGeom g;
  int muon;
  const float* gx0; const void* g16; const float* norms; const float* dot_part; int nparts;
  const float* gw_hat; float cr;     // added when the raw gradient also enters w_hat
  float* gm_carry; int carry_valid;  // gradient w.r.t. the momentum state after this update (in/out)
  const float* m_prev; const float* mbar;   // null without momentum
  void* gc;                          // [3b][elems] compute-type copy of d loss / d dw  (GEMM operand)
  uint16_t* gct;                     // bf16 transposed copy ([cols][rows]) or null
  float* mdot_part;                  // [3b][gridDim.x] partial <g, m_prev>
};
template <typename T, typename TN>
__global__ void k_grad_prep(const GradPrepParams p) {
  __shared__ float red[16];
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  float c0 = 1.f, c1 = 0.f;
  if (p.muon) {
    float dot = 0.f;
    for (int i = 0; i < p.nparts; ++i) dot += p.dot_part[(size_t)z * p.nparts + i];
    const float n = p.norms[z];
    c0 = 1.f / (n + 1e-7f);
    c1 = n > 0.f ? dot / (n * (n + 1e-7f) * (n + 1e-7f)) : 0.f;
  }
  const float mb = p.mbar ? p.mbar[ib] : 0.f;
  const long long per = (p.g.elems + gridDim.x - 1) / gridDim.x;
  const long long e0 = blockIdx.x * per, e1 = min(e0 + per, p.g.elems);
  float md = 0.f;
  for (long long e = e0 + threadIdx.x; e < e1; e += blockDim.x) {
    const size_t o = (size_t)z * p.g.elems + e;
    float gv;
    if (p.muon) {
      const size_t x = (size_t)z * p.g.elems + p.g.xidx(j, e);
      gv = p.gx0[x] * c0 - Elem<TN>::load(reinterpret_cast<const TN*>(p.g16) + x) * c1;
      if (p.cr != 0.f) gv += p.cr * p.gw_hat[o];
    } else {
      gv = p.gw_hat[o];
    }
    if (p.gm_carry) {
      if (p.carry_valid) gv += p.gm_carry[o];
      p.gm_carry[o] = gv * mb;                       // d/d M_prev of  dw + M_prev * mbar
      if (p.m_prev) md += gv * p.m_prev[o];
    }
    Elem<T>::store(reinterpret_cast<T*>(p.gc) + o, gv);
    if (p.gct) {
      const int cols = p.g.cols(j);
      p.gct[(size_t)z * p.g.elems + (e % cols) * p.g.rows(j) + e / cols] = f32_to_bf16(gv);
    }
  }
  if (p.gm_carry) {
    md = block_sum(md, red);
    if (threadIdx.x == 0) p.mdot_part[(size_t)z * gridDim.x + blockIdx.x] = md;
  }
}

// d loss / d momentum[t] = <g, M_prev> / chunk_len for every token of the chunk (mean, :172)
__global__ void k_momentum_grad(const float* mdot_part, int nparts, int nb, float* dmom, long long bs, int start, int len) {
  const int ib = blockIdx.x;
  float s = 0.f;
  for (int j = 0; j < 3; ++j)
    for (int i = 0; i < nparts; ++i) s += mdot_part[(size_t)(j * nb + ib) * nparts + i];
  s /= (float)len;
  for (int t = threadIdx.x; t < len; t += blockDim.x) dmom[ib * bs + start + t] += s;
}

// out = coeff*in_add + sum of split partials
__global__ void k_reduce_partials(float* out, const float* in_add, float coeff, const float* partial, int nsplit, long long total) {
  const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= total) return;
  float v = in_add ? coeff * in_add[e] : 0.f;
  for (int s = 0; s < nsplit; ++s) v += partial[(size_t)s * total + e];
  out[e] = v;
}

// dlr_j[ib, start + t] += sum over slots of the row partials
__global__ void k_lr_reduce(const float* lrpart, long long mat_stride, long long slot_stride, int nslots, int Tcap,
                            float* dlr0, float* dlr1, float* dlr2, long long bs, int start, int len) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x, ib = blockIdx.y, j = blockIdx.z;
  if (t >= len) return;
  float s = 0.f;
  for (int i = 0; i < nslots; ++i) s += lrpart[j * mat_stride + i * slot_stride + (size_t)ib * Tcap + t];
  float* dst = j == 0 ? dlr0 : (j == 1 ? dlr1 : dlr2);
  dst[ib * bs + start + t] += s;
}

// final weight gradients: state gradient (+ accumulator carry) + the path through the initial row norms
struct FinishParams {
  MatGeom g;
  const float* gw; const float* carry; const float* gn0; const float* n0; const float* w_init;
  int through_norms;
  float* out[3];
};
__global__ void k_finish_weight_grads(const FinishParams p) {
  const int z = blockIdx.y, j = z / p.g.nb, ib = z % p.g.nb;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= p.g.rows(j)) return;
  const int cols = p.g.cols(j);
  const size_t o = (size_t)z * p.g.elems + (size_t)row * cols;
  float c = 0.f;
  if (p.through_norms) {
    const float n = p.n0[(size_t)z * p.g.maxrows() + row];
    c = n > 0.f ? p.gn0[(size_t)z * p.g.maxrows() + row] / n : 0.f;
  }
  float* dst = p.out[j] + (size_t)ib * p.g.elems + (size_t)row * cols;
  for (int k = lane; k < cols; k += 64) {
    float v = p.gw[o + k];
    if (p.carry) v += p.carry[o + k];
    if (p.through_norms) v += c * p.w_init[o + k];
    dst[k] = v;
  }
}

// unpack [3b][elems] into the three caller tensors
__global__ void k_unpack3(const float* src, long long elems, int nb, float* o0, float* o1, float* o2) {
  const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const int z = blockIdx.y;
  if (e >= elems) return;
  float* dst = (z / nb) == 0 ? o0 : ((z / nb) == 1 ? o1 : o2);
  if (dst) dst[(size_t)(z % nb) * elems + e] = src[(size_t)z * elems + e];
}
__global__ void k_pack3(float* dst, long long elems, int nb, const float* i0, const float* i1, const float* i2) {
  const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const int z = blockIdx.y;
  if (e >= elems) return;
  const float* src = (z / nb) == 0 ? i0 : ((z / nb) == 1 ? i1 : i2);
  dst[(size_t)z * elems + e] = src ? src[(size_t)(z % nb) * elems + e] : 0.f;
}
// dst[z][c*rows + r] = src[z][r*cols + c] for bf16 matrices; kind j = z / nb picks (rows, cols).
struct TransposeParams {
  const uint16_t* src; uint16_t* dst;
  int rows[3], cols[3];
  int nb; long long elems;
};
__global__ __launch_bounds__(256) void k_transpose_b16(const TransposeParams p) {
  __shared__ uint16_t tile[64][66];
  const int z = blockIdx.z, j = z / p.nb;
  const int rows = p.rows[j], cols = p.cols[j];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  if (r0 >= rows || c0 >= cols) return;
  const uint16_t* src = p.src + (size_t)z * p.elems;
  uint16_t* dst = p.dst + (size_t)z * p.elems;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = threadIdx.x + i * 256, r = idx / 16, c = (idx % 16) * 4;
    uint2 v = make_uint2(0, 0);
    if (r0 + r < rows && c0 + c < cols) v = *reinterpret_cast<const uint2*>(src + (size_t)(r0 + r) * cols + c0 + c);
    tile[r][c] = (uint16_t)(v.x & 0xffff); tile[r][c + 1] = (uint16_t)(v.x >> 16);
    tile[r][c + 2] = (uint16_t)(v.y & 0xffff); tile[r][c + 3] = (uint16_t)(v.y >> 16);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = threadIdx.x + i * 256, c = idx / 16, r = (idx % 16) * 4;
    if (c0 + c < cols && r0 + r < rows) {
      uint2 v;
      v.x = (uint32_t)tile[r][c] | ((uint32_t)tile[r + 1][c] << 16);
      v.y = (uint32_t)tile[r + 2][c] | ((uint32_t)tile[r + 3][c] << 16);
      *reinterpret_cast<uint2*>(dst + (size_t)(c0 + c) * rows + r0 + r) = v;
    }
  }
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
