// Persistent bf16 tile engine: a block walks a list of output tiles; the copy waves never stop at a tile boundary.
//
//   matrix waves  (0-3): fragments from the LDS ring, MFMAs, and at the end of a tile its epilogue, straight from the
//                        accumulators;
//   service waves (4-7): the asynchronous global -> LDS copies of the ring, in one flat sequence over all phases of all
//                        tiles of the block: while the matrix waves run a tile's epilogue, the next tile's first two
//                        stages are already landing.
//
// Why this pays: with one tile per block the ring's fill, the epilogue and the dispatcher's lock-step rounds are paid in
// line, copy engine idle; here the next tile's fill hides behind the epilogue.  What it does not change is the main
// loop itself: a 48 KiB K-step takes 0.75-1 us to copy against 0.43 us of matrix work (measured with the matrix work and
// the epilogue switched off: the copies alone take 18-20 us of a 33 us launch at 18 K-steps per block).
//
// Measured and rejected on the way:
//   * the epilogue on the copy waves, fed through LDS (hand-over of the rounded accumulators), to run it "beside" the
//     matrix work -- a wave stalls in order while its copy instructions wait for the address queue, so a copy wave
//     cannot compute during the copies it issues, and every epilogue instruction it executes delays the next stage:
//     apply 37.3 us per launch against 37.4 for one tile per block, update 150 against 92;
//   * the matrix waves touching every 128-byte line of the next tile's token rows a tile ahead (one 4-byte asynchronous
//     copy per line into an LDS area nobody reads), so that the rows are in the L2 when their copies run: apply 36.6 us
//     against 34.0, apply backward 65.5 against 59.2 -- the touches cost a stage's worth of address processing per tile
//     and the copies behind them are no faster;
//   * all hidden tiles of a token tile on one block, back to back, so that the token rows come from HBM once and from
//     the L2 twice: apply 36.6 us against 33.4, apply backward 62.5 against 58.2 (three blocks that fetch the same rows
//     at the same moment share one HBM fetch just as well).
//
// Epilogue stores.  A lane owns 4 consecutive columns of 32 different rows per 32 x 32 fragment; stored straight from
// the accumulators that is 32 cache lines per instruction.  The ring slot of the tile's last K-step is free once every
// matrix wave is past its last fetch (one block barrier): each matrix wave stages up to six fragments of results there
// as [32 rows][64 bytes], reads them back row-wise (4 lanes x 16 bytes per row) and stores 64-byte row segments, all
// reads of a group before its stores.  The part of the slot a wave uses is its own and the LDS operations of a wave
// execute in order: no further barrier.  The copy waves refill that slot only after the next tile's first barrier.
#pragma once
#include <algorithm>

#include "gemm_dma_kernels.h"

namespace lact {

constexpr int PS_STAGES = 3;

// s_waitcnt vmcnt(n) for a wave-uniform run-time n.  The immediate must be a constant, so n is rounded DOWN to a
// multiple of four (a smaller count only waits longer; the copy waves issue copies in fours) and a short chain of scalar
// branches picks it.  The chain is on the copy waves' critical path once per K-step: a wave issues an instruction
// every four or five cycles at best and a taken branch costs a few times that, so a 64-leaf tree here cost 1-2 us per
// launch.
__device__ __forceinline__ void wait_vmcnt_dyn(int n) {
  n = __builtin_amdgcn_readfirstlane(n);
  if (n >= 12) {
    if (n >= 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else if (n >= 20) asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
    else if (n >= 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
  } else {
    if (n >= 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (n >= 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
}

// ---- tile list of a block: tiles b, b + G, b + 2 G, ... of the launch's tile map (G = grid, a multiple of 8: all of a
// block's tiles belong to the XCD the map assumes for it)
struct TileWalk {
  int next, stride, end;
  __device__ __forceinline__ void init(int grid_tiles) { next = blockIdx.x; stride = gridDim.x; end = grid_tiles; }
  __device__ __forceinline__ bool take(int& lin) {
    if (next >= end) return false;
    lin = next;
    next += stride;
    return true;
  }
};
// blocks of a persistent launch over `tiles` tiles (tiles a multiple of 8) on a device with `cus` compute units
inline int persist_grid(int tiles, int cus) {
  const int per = (tiles + cus - 1) / cus;
  const int blocks = (tiles + per - 1) / per;
  return std::min(tiles, 8 * ((blocks + 7) / 8));
}

// ---- epilogue window: one 32 x 32 bf16 fragment per matrix wave at a time -------------------------------------------
// [32 rows][64 bytes]; the 16-byte granule j of row r sits at slot j ^ ((r >> 2) & 3) (two-way bank conflicts on the
// 8-byte writes, four-way on the 16-byte reads: both the minimum for their width).
constexpr int FRAG_BYTES = 32 * 64;
constexpr int WAVE_FRAGS = 6;                      // fragments a matrix wave stages at a time
constexpr int WINDOW_BYTES = 4 * WAVE_FRAGS * FRAG_BYTES;   // 48 KiB: one ring slot of a two-operand 128 x 128 stage

// the four values (columns 8 g + 4 h + 0..3 of row m; m = lane & 31, h = lane >> 5) of this lane, packed, into `frag`
__device__ __forceinline__ void frag_put(char* frag, int g, uint32_t lo, uint32_t hi) {
  const int l = threadIdx.x & 63, m = l & 31, h = l >> 5;
  *reinterpret_cast<uint2*>(frag + m * 64 + ((g ^ ((m >> 2) & 3)) << 4) + h * 8) = make_uint2(lo, hi);
}
__device__ __forceinline__ void frag_put4(char* frag, int g, float a, float b, float c, float d) {
  frag_put(frag, g, (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16), (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16));
}
// the fragment back, row-wise: lane l holds columns [8 (l & 3), + 8) of rows (l >> 2) and (l >> 2) + 16
__device__ __forceinline__ void frag_read(const char* frag, uint4 (&v)[2]) {
  const int l = threadIdx.x & 63, j = l & 3;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int r = (l >> 2) + 16 * p;
    v[p] = *reinterpret_cast<const uint4*>(frag + r * 64 + ((j ^ ((r >> 2) & 3)) << 4));
  }
}
// ... and to `out` (first element of the fragment, row stride ld elements); rows / cols = valid extent from the fragment's origin
__device__ __forceinline__ void frag_store(const uint4 (&v)[2], uint16_t* out, int ld, int rows, int cols) {
  const int l = threadIdx.x & 63, j = l & 3;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int r = (l >> 2) + 16 * p;
    if (r < rows && 8 * j < cols) *reinterpret_cast<uint4*>(out + (size_t)r * ld + 8 * j) = v[p];
  }
}

// ---- service side: the copy cursor ------------------------------------------------------------------------------------
// Issues the ring's stages in order over the phases of a tile and on into the next tile's, and keeps the count of
// vector-memory operations this wave has issued, from which the wait for a stage derives its vmcnt.
template <class TS, int NB, int NPH>
struct CopyCursor {
  using SM = DmaSmem<TS, NB, PS_STAGES>;
  char* smem;
  int lw;
  DmaLane<TS::BM> la;
  DmaLane<TS::BN> lb[NB];
  DmaPhase<NB> ph[NPH];
  int cp, ckt, cnk, cnb;
  int issued;               // stages issued so far (all tiles)
  bool valid;               // the cursor points at a stage that exists
  int ops;                  // vector-memory operations issued by this wave so far
  // value of `ops` right after the copies of each stage that has been issued and not yet waited for (oldest first);
  // scalars, not an array: an indexed array would live in scratch memory, whose loads drain the copy queue
  int mark0, mark1, mark2, nmarks;
  int islot;                // ring slot of the next stage to issue

  __device__ __forceinline__ void init(char* s) {
    smem = s;
    lw = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) - 4;
    issued = 0; ops = 0; valid = false; cp = NPH - 1; ckt = 0; cnk = 0; cnb = 0;
    mark0 = mark1 = mark2 = 0; nmarks = 0; islot = 0;
  }
  __device__ __forceinline__ void select_phase() {
#pragma unroll
    for (int i = 0; i < NPH; ++i)
      if (i == cp) {
        la.init(ph[i].a, lw);
#pragma unroll
        for (int j = 0; j < NB; ++j) lb[j].init(ph[i].b[j], lw);
        cnb = ph[i].nb;
        cnk = ph[i].K / DMA_BK;
      }
    ckt = 0;
  }
  // next(ph, ops) fills the phases of the following tile; returns false when there is no further tile
  template <class Next>
  __device__ __forceinline__ void advance(Next& next) {
    valid = false;
    for (int tries = 0; tries <= NPH; ++tries) {   // a tile has at least one phase with K-steps
      ++cp;
      if (cp >= NPH) {
        if (!next(ph, ops)) return;
        cp = 0;
      }
      select_phase();
      if (cnk > 0) { valid = true; return; }
    }
  }
  template <class Next>
  __device__ __forceinline__ void issue_stage(Next& next) {
    const uint32_t base = lds_addr(smem + islot * SM::STAGE) + lw * 1024;
    la.template issue<false>(ckt, base);
#pragma unroll
    for (int j = 0; j < NB; ++j)
      if (j < cnb) lb[j].template issue<false>(ckt, base + SM::A_BYTES + j * SM::B_BYTES);
    ops += (TS::BM + cnb * TS::BN) / 8 / DMA_LOADERS;
    if (nmarks == 0) mark0 = ops;
    else if (nmarks == 1) mark1 = ops;
    else mark2 = ops;
    ++nmarks;
    islot = islot == PS_STAGES - 1 ? 0 : islot + 1;
    ++issued;
    if (++ckt == cnk) advance(next);
  }
  // the oldest stage that has been issued and not waited for has landed in its slot
  __device__ __forceinline__ void wait_oldest_stage() {
    wait_vmcnt_dyn(ops - mark0);
    mark0 = mark1; mark1 = mark2; --nmarks;
  }
};

// ------------------------------------------------------------------------------------------------------------------
// Hidden-stage kernels on the persistent engine.  TS = 128 x 128, waves 2 x 2 (64 x 64 per wave, TM = TN = 2).
// ------------------------------------------------------------------------------------------------------------------
struct HiddenPersistParams {
  HiddenParams h;
  TileMap map;    // token tiles, hidden tiles, batch
};

// Where a matrix wave's fragment (tm, tn) lies: origin inside the tile and the valid extent from there.
struct FragPlace {
  int m0, n0, z, T, dh;       // tile origin, batch entry, problem extent
  int wrow, wcol;             // this wave's 64 x 64 part of the tile
  char* win;                  // this wave's two fragment buffers
  __device__ __forceinline__ void init(char* window, int m0_, int n0_, int z_, int T_, int dh_) {
    const int w = threadIdx.x >> 6;
    m0 = m0_; n0 = n0_; z = z_; T = T_; dh = dh_;
    wrow = (w / 2) * 64; wcol = (w % 2) * 64;
    win = window + w * WAVE_FRAGS * FRAG_BYTES;
  }
  __device__ __forceinline__ int row(int tm) const { return m0 + wrow + tm * 32; }
  __device__ __forceinline__ int col(int tn) const { return n0 + wcol + tn * 32; }
  __device__ __forceinline__ char* buf(int b) const { return win + b * FRAG_BYTES; }
  // buffers b0 .. b0 + N - 1 hold fragment (tm, tn) of the [T, dh] arrays outs[0 .. N - 1] (batch stride bs elements):
  // all reads first, then all stores
  template <int N>
  __device__ __forceinline__ void flush(int b0, void* const (&outs)[N], long long bs, int tm, int tn) const {
    const int r = row(tm), c = col(tn);
    uint4 v[N][2];
#pragma unroll
    for (int i = 0; i < N; ++i) frag_read(buf(b0 + i), v[i]);
#pragma unroll
    for (int i = 0; i < N; ++i)
      frag_store(v[i], reinterpret_cast<uint16_t*>(outs[i]) + z * bs + (size_t)r * dh + c, dh, T - r, dh - c);
  }
};

// Kernel policies: phases() for the copy waves, mma() and epilogue() for the matrix waves.

// apply forward: O0 = silu(X W0^T) * (X W2^T)
struct ApplyHiddenPolicy {
  static constexpr int NACC = 2, NB = 2, NPH = 1;
  using TS = TS_SQ;
  __device__ static __forceinline__ void phases(const HiddenParams& p, int m0, int n0, int z, DmaPhase<2> (&ph)[1]) {
    ph[0].a = token_operand<TS>(p.X, p.bsx, p.ldx, z, m0, p.T);
    ph[0].b[0] = weight_operand(p.W0, p.bsw, p.d, z, n0, p.dh);
    ph[0].b[1] = weight_operand(p.W2, p.bsw, p.d, z, n0, p.dh);
    ph[0].nb = 2;
    ph[0].K = p.d;
  }
  template <class Pipe>
  __device__ static __forceinline__ void mma(Pipe& pipe, const HiddenParams& p, int& step, f32x16 (&a02)[2][2][2], f32x16 (&)[1][2][2]) {
    pipe.template run_phase<2>(p.d / DMA_BK, step, a02);
  }
  __device__ static __forceinline__ void epilogue(const HiddenParams& p, const FragPlace& f, const f32x16 (&a02)[2][2][2], const f32x16 (&)[1][2][2]) {
    // all four fragments of the wave staged, then stored
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float y0 = round_bf16(a02[0][tm][tn][4 * g + j]), y2 = round_bf16(a02[1][tm][tn][4 * g + j]);
            v[j] = round_bf16(y0 * sigmoidf_(y0)) * y2;
          }
          frag_put4(f.buf(tm * 2 + tn), g, v[0], v[1], v[2], v[3]);
        }
    void* const o[1] = {p.O0};
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int tn = 0; tn < 2; ++tn) f.flush<1>(tm * 2 + tn, o, p.bso, tm, tn);
  }
};

// apply backward, hidden stage: O0 = hidden (recomputed), O1 = d/d(X W0^T), O2 = d/d(X W2^T); Y = upstream gradient
struct ApplyBwdHiddenPolicy {
  static constexpr int NACC = 3, NB = 2, NPH = 2;
  using TS = TS_SQ;
  __device__ static __forceinline__ void phases(const HiddenParams& p, int m0, int n0, int z, DmaPhase<2> (&ph)[2]) {
    ph[0].a = token_operand<TS>(p.X, p.bsx, p.ldx, z, m0, p.T);
    ph[0].b[0] = weight_operand(p.W0, p.bsw, p.d, z, n0, p.dh);
    ph[0].b[1] = weight_operand(p.W2, p.bsw, p.d, z, n0, p.dh);
    ph[0].nb = 2;
    ph[0].K = p.d;
    ph[1].a = token_operand<TS>(p.Y, p.bsy, p.ldy, z, m0, p.T);
    ph[1].b[0] = weight_operand_ks(p.W1, p.bsw, p.dh, z, n0, p.dh);
    ph[1].b[1] = ph[1].b[0];
    ph[1].nb = 1;
    ph[1].K = p.d;
  }
  template <class Pipe>
  __device__ static __forceinline__ void mma(Pipe& pipe, const HiddenParams& p, int& step, f32x16 (&a02)[2][2][2], f32x16 (&a1)[1][2][2]) {
    pipe.template run_phase<2>(p.d / DMA_BK, step, a02);
    pipe.template run_phase<1, false, true>(p.d / DMA_BK, step, a1);
  }
  __device__ static __forceinline__ void epilogue(const HiddenParams& p, const FragPlace& f, const f32x16 (&a02)[2][2][2], const f32x16 (&a1)[1][2][2]) {
    void* const o[3] = {p.O0, p.O1, p.O2};
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
      // the three outputs of both fragments of this row block staged (six buffers), then stored
#pragma unroll
      for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float hq[4], gy0[4], gy2[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float y0 = round_bf16(a02[0][tm][tn][4 * g + j]), y2 = round_bf16(a02[1][tm][tn][4 * g + j]);
            const float gh = round_bf16(a1[0][tm][tn][4 * g + j]);
            const SiluParts s = silu_parts(y0);
            const float sg = round_bf16(s.silu);
            hq[j] = sg * y2; gy0[j] = round_bf16(gh * y2) * s.d1; gy2[j] = gh * sg;
          }
          frag_put4(f.buf(tn * 3 + 0), g, hq[0], hq[1], hq[2], hq[3]);
          frag_put4(f.buf(tn * 3 + 1), g, gy0[0], gy0[1], gy0[2], gy0[3]);
          frag_put4(f.buf(tn * 3 + 2), g, gy2[0], gy2[1], gy2[2], gy2[3]);
        }
#pragma unroll
      for (int tn = 0; tn < 2; ++tn) f.flush<3>(tn * 3, o, p.bso, tm, tn);
    }
  }
};

// update forward: O0 = dgate_before_act, O1 = hidden * lr1, O2 = dhidden_before_mul (the operands of the three fast-weight
// gradient GEMMs: lr0 and lr2 scale k there, ttt_operation.py:166-168).  For the backward, when O3 is set: O3..O5 = the
// rounded pre-activations, O6 = O0 * lr0, O7 = O2 * lr2.
struct UpdateHiddenPolicy {
  static constexpr int NACC = 3, NB = 2, NPH = 2;
  using TS = TS_SQ;
  __device__ static __forceinline__ void phases(const HiddenParams& p, int m0, int n0, int z, DmaPhase<2> (&ph)[2]) {
    ApplyBwdHiddenPolicy::phases(p, m0, n0, z, ph);
  }
  template <class Pipe>
  __device__ static __forceinline__ void mma(Pipe& pipe, const HiddenParams& p, int& step, f32x16 (&a02)[2][2][2], f32x16 (&a1)[1][2][2]) {
    ApplyBwdHiddenPolicy::mma(pipe, p, step, a02, a1);
  }
  __device__ static __forceinline__ void epilogue(const HiddenParams& p, const FragPlace& f, const f32x16 (&a02)[2][2][2], const f32x16 (&a1)[1][2][2]) {
    const bool keep = p.O3 != nullptr;
    void* const o3[3] = {p.O0, p.O1, p.O2};
    void* const o5[5] = {p.O0, p.O1, p.O2, p.O6, p.O7};
    void* const opre[3] = {p.O3, p.O4, p.O5};
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
      const int m = f.row(tm) + (threadIdx.x & 31);
      const bool mv = m < p.T;
      const float l0 = mv ? p.lr0[f.z * p.bslr + m] : 0.f, l1 = mv ? p.lr1[f.z * p.bslr + m] : 0.f;
      const float l2 = mv ? p.lr2[f.z * p.bslr + m] : 0.f;
#pragma unroll
      for (int tn = 0; tn < 2; ++tn) {
        // one fragment of the five computed outputs staged (buffers 0-4), stored; then the three rounded pre-activations
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float o[5][4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float gg = round_bf16(a02[0][tm][tn][4 * g + j]), h2 = round_bf16(a02[1][tm][tn][4 * g + j]);
            const float dh = round_bf16(a1[0][tm][tn][4 * g + j]);
            const UpdatePointwise u = update_pointwise<uint16_t>(gg, h2, dh, silu_parts(gg));
            o[0][j] = u.dgpre; o[1][j] = u.hid * l1; o[2][j] = u.dh2;
            o[3][j] = u.dgpre * l0; o[4][j] = u.dh2 * l2;
          }
#pragma unroll
          for (int k = 0; k < 5; ++k) frag_put4(f.buf(k), g, o[k][0], o[k][1], o[k][2], o[k][3]);
        }
        if (keep) f.flush<5>(0, o5, p.bso, tm, tn);
        else f.flush<3>(0, o3, p.bso, tm, tn);
        if (keep) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            frag_put4(f.buf(0), g, a02[0][tm][tn][4 * g], a02[0][tm][tn][4 * g + 1], a02[0][tm][tn][4 * g + 2], a02[0][tm][tn][4 * g + 3]);
            frag_put4(f.buf(1), g, a02[1][tm][tn][4 * g], a02[1][tm][tn][4 * g + 1], a02[1][tm][tn][4 * g + 2], a02[1][tm][tn][4 * g + 3]);
            frag_put4(f.buf(2), g, a1[0][tm][tn][4 * g], a1[0][tm][tn][4 * g + 1], a1[0][tm][tn][4 * g + 2], a1[0][tm][tn][4 * g + 3]);
          }
          f.flush<3>(0, opre, p.bso, tm, tn);
        }
      }
    }
  }
};

// ---- the kernel --------------------------------------------------------------------------------------------------------
template <class POL>
struct PersistLds {
  using SM = DmaSmem<typename POL::TS, POL::NB, PS_STAGES>;
  static constexpr int RING = SM::BYTES;
  static constexpr int BYTES = RING;
  static_assert(SM::STAGE >= WINDOW_BYTES, "the epilogue window is the ring slot of a tile's last K-step");
};

// What the copy cursor does when it enters a new tile: the tile's phases.
template <class POL>
struct NextHiddenTile {
  using TS = typename POL::TS;
  const HiddenPersistParams* pp;
  TileWalk walk;
  __device__ __forceinline__ bool operator()(DmaPhase<POL::NB> (&ph)[POL::NPH], int&) {
    int lin, bx, by, z;
    while (walk.take(lin)) {
      if (!pp->map.locate(lin, bx, by, z)) continue;
      POL::phases(pp->h, bx * TS::BM, by * TS::BN, z, ph);
      return true;
    }
    return false;
  }
};

template <class POL>
__global__ __launch_bounds__(DMA_THREADS) void k_hidden_persist(const HiddenPersistParams pp) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  using TS = typename POL::TS;
  using L = PersistLds<POL>;
  static_assert(TS::BM == 128 && TS::BN == 128 && TS::WM == 64 && TS::WN == 64, "64 x 64 per wave");
  const HiddenParams& p = pp.h;
  const bool service = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) >= 4;
  // K-steps of a tile (the same for every tile of the launch)
  int nk_tile;
  {
    DmaPhase<POL::NB> ph0[POL::NPH];
    POL::phases(p, 0, 0, 0, ph0);
    nk_tile = 0;
#pragma unroll
    for (int i = 0; i < POL::NPH; ++i) nk_tile += ph0[i].K / DMA_BK;
  }
  if (nk_tile <= 0) return;

  if (service) {
    // ------------------------------------------------------------------------------------------ service waves
    CopyCursor<TS, POL::NB, POL::NPH> cur;
    cur.init(smem);
    NextHiddenTile<POL> next_tile;
    next_tile.pp = &pp;
    next_tile.walk.init(pp.map.grid());
    cur.advance(next_tile);
    TileWalk walk;           // tiles as they are consumed
    walk.init(pp.map.grid());
    int g = 0;               // K-steps consumed so far (all tiles)
    for (int i = 0; i < PS_STAGES - 1 && cur.valid; ++i) cur.issue_stage(next_tile);
    int lin;
    while (walk.take(lin)) {
      int bx, by, z;
      if (!pp.map.locate(lin, bx, by, z)) continue;
      for (int kt = 0; kt < nk_tile; ++kt, ++g) {
        // stage g landed -> barrier -> refill the slot the matrix waves have left
        cur.wait_oldest_stage();
        __syncthreads();
        if (cur.valid && cur.issued <= g + PS_STAGES - 1) cur.issue_stage(next_tile);
      }
      // the matrix waves' end-of-loop barrier.  The slot of the tile's last K-step is their epilogue window until they
      // reach the next tile's first barrier: two stages of the next tile are in flight meanwhile.
      __syncthreads();
    }
  } else {
    // ------------------------------------------------------------------------------------------- matrix waves
    using Pipe = DmaPipe<TS, POL::NB, POL::NPH, PS_STAGES>;
    DmaPhase<POL::NB> phd[POL::NPH];
    POL::phases(p, 0, 0, 0, phd);
    Pipe pipe(smem, phd);
    TileWalk walk;
    walk.init(pp.map.grid());
    int step = 0, lin;
    f32x16 a02[2][2][2], a1[1][2][2];
    FragPlace f;
    while (walk.take(lin)) {
      int bx, by, z;
      if (!pp.map.locate(lin, bx, by, z)) continue;
      zero_acc<TS>(a02[0]);
      zero_acc<TS>(a02[1]);
      if (POL::NACC > 2) zero_acc<TS>(a1[0]);
      POL::mma(pipe, p, step, a02, a1);
      // Window: the slot of the K-step just finished.  Every matrix wave read fragments from all of it, so all of them
      // must be past their last fetch before any of them writes there: one barrier (the copy waves join it).
      __syncthreads();
      f.init(smem + ((step - 1) % PS_STAGES) * L::SM::STAGE, bx * TS::BM, by * TS::BN, z, p.T, p.dh);
      POL::epilogue(p, f, a02, a1);
    }
  }
}

}  // namespace lact
