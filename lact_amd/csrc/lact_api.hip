// Host side of liblact_hip.so: validates a program, lays out the caller's buffers and enqueues the
// kernels of the forward and backward passes on the caller's stream.  No allocation, no
// synchronisation, no torch types.
#include "../../include/lact_hip.h"

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>
#include <mutex>
#include <memory>

#include <type_traits>

#include "gemm_dma_kernels.h"
#include "ns_fused.h"
#include "gemm_persist.h"
#include "gemm_kernels.h"
#include "state_kernels.h"
#include "layer_kernels.h"

using namespace lact;

namespace {

thread_local std::string g_err;
int fail(const std::string& m) {
  g_err = m;
  return -1;
}
// ---- optional per-launch timing (HIP events on the caller's stream) ---------------------------------
struct ProfRec {
  const char* kernel;
  const char* site;
  double flops;
  hipEvent_t e0, e1;
};
struct Profiler {
  bool on = false;
  std::vector<ProfRec> recs;
  std::vector<hipEvent_t> pool;
  hipEvent_t get() {
    if (!pool.empty()) {
      hipEvent_t e = pool.back();
      pool.pop_back();
      return e;
    }
    hipEvent_t e;
    (void)hipEventCreate(&e);
    return e;
  }
  void clear() {
    for (auto& r : recs) {
      pool.push_back(r.e0);
      pool.push_back(r.e1);
    }
    recs.clear();
  }
};
Profiler g_prof;
struct ProfScope {
  hipStream_t s;
  hipEvent_t e1 = nullptr;
  ProfScope(const char* kernel, const char* site, double flops, hipStream_t st) : s(st) {
    if (!g_prof.on) return;
    ProfRec r{kernel, site, flops, g_prof.get(), g_prof.get()};
    (void)hipEventRecord(r.e0, s);
    e1 = r.e1;
    g_prof.recs.push_back(r);
  }
  ~ProfScope() {
    if (e1) (void)hipEventRecord(e1, s);
  }
};
// kern may contain template commas: pass it parenthesised
#define LACT_LAUNCH(kname, site, flops, kern, grid, block, stream, ...)  \
  do {                                                                  \
    ProfScope ps_(kname, site, flops, stream);                          \
    hipLaunchKernelGGL(kern, grid, block, 0, stream, __VA_ARGS__);      \
  } while (0)

#define LACT_LAUNCH_SMEM(kname, site, flops, kern, grid, block, smem_bytes, stream, ...) \
  do {                                                                                   \
    ProfScope ps_(kname, site, flops, stream);                                           \
    hipLaunchKernelGGL(kern, grid, block, smem_bytes, stream, __VA_ARGS__);              \
  } while (0)

// Kernels whose ring exceeds the default dynamic LDS limit opt in once per call site (= instantiation) and device:
// the attribute belongs to the current device.
inline void allow_big_lds(std::atomic<uint64_t>& done, const void* kern, int bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  const uint64_t bit = 1ull << dev;
  if (done.load(std::memory_order_acquire) & bit) return;
  (void)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  done.fetch_or(bit, std::memory_order_release);
}
#define LACT_BIG_LDS(kern, bytes)                                         \
  do {                                                                    \
    static std::atomic<uint64_t> done_{0};                                \
    allow_big_lds(done_, reinterpret_cast<const void*>(kern), bytes);     \
  } while (0)

template <typename T> const char* tname();
template <> const char* tname<uint16_t>() { return "bf16"; }
template <> const char* tname<float>() { return "f32"; }

#define LACT_CHECK_LAUNCH()                                                     \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) return fail(std::string("kernel launch failed: ") + hipGetErrorString(e_)); \
  } while (0)

// ---- side stream: the apply steps of a program do not depend on the update chain that runs beside them
// (block-causal: apply(i) and update(i) both read weight version i), so they are enqueued on a second
// stream of default priority, forked from and joined back into the caller's stream with events.  The
// memory-bound tails of one chain then overlap the matrix work of the other.  One stream and one event
// pool per device, created on first use and kept until the process ends.
struct SideCtx {
  hipStream_t stream = nullptr;
  hipStream_t tail = nullptr;        // second side stream: results of the update chain that nothing in the call waits for
  std::vector<hipEvent_t> ev;
  size_t next = 0;
  // Fused Newton-Schulz kernels of this process must not overlap each other (each needs its groups resident as a whole).
  // Launches on one stream follow each other anyway; an event is recorded (on the stream of the newest launch, at the
  // time the next launch arrives) only when that next launch comes from another stream -- a record behind every launch
  // would put ~3 us between the kernel and whatever follows it on the caller's stream.
  hipEvent_t fused_done = nullptr;
  hipStream_t fused_stream = nullptr;
  bool fused_any = false;
  void order_fused_launch(hipStream_t s) {
    if (fused_any && fused_stream != s) {
      if (!fused_done) (void)hipEventCreateWithFlags(&fused_done, hipEventDisableTiming);
      if (hipEventRecord(fused_done, fused_stream) == hipSuccess) {
        (void)hipStreamWaitEvent(s, fused_done, 0);
      } else {   // that stream no longer exists: whatever it still runs is waited for the hard way
        (void)hipGetLastError();
        (void)hipDeviceSynchronize();
      }
    }
    fused_stream = s;
    fused_any = true;
  }
  int cus = 0;                       // compute units of the device (0: not asked yet)
  unsigned* sticky = nullptr;        // device address of this device's count of barrier time-outs
  hipEvent_t event() {
    if (next == ev.size()) {
      hipEvent_t e;
      (void)hipEventCreateWithFlags(&e, hipEventDisableTiming);
      ev.push_back(e);
    }
    return ev[next++];
  }
};
}  // namespace
// Barrier waits of the fused Newton-Schulz kernels that gave up, counted per device since the last
// lact_check_async_error (each GPU holds its own copy; host code reaches it through hipGetSymbolAddress only).
static __device__ unsigned g_async_errors;
namespace {
bool g_overlap = true;
bool g_fused_ns = true;
int g_keep_pre = -1;       // LACT_OPT_KEEP_PREACTIVATIONS: -1 by shape, 0 never, 1 whenever the kernels allow it
int g_persist = 1;          // hidden-stage kernels on the persistent engine (LACT_OPT_PERSISTENT_TILES): bit 0 apply, 1 update, 2 apply backward
                            // (the one-tile-per-block kernels of the update and the apply backward, whose pointwise epilogues run on all
                            // eight waves, measured faster than their persistent versions: only the apply's is on by default)
long long g_ns_spin_limit = NS_FUSED_SPIN_LIMIT;   // barrier wait bound of the fused Newton-Schulz kernels (lact_set_option)
std::mutex g_enqueue_mutex;   // one program is enqueued at a time (the side-stream context is shared)
SideCtx* side_ctx() {
  static SideCtx ctx[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  SideCtx& c = ctx[dev];
  if (!c.stream && hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking) != hipSuccess) return nullptr;
  if (!c.tail && hipStreamCreateWithFlags(&c.tail, hipStreamNonBlocking) != hipSuccess) return nullptr;
  if (c.cus == 0) {
    int n = 0;
    c.cus = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : -1;
  }
  if (!c.sticky) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_async_errors)) == hipSuccess) c.sticky = static_cast<unsigned*>(ptr);
  }
  c.next = 0;
  return &c;
}

using TSA = TileShape<128, 128, 2, 2>;  // two or three accumulators
using TSB = TileShape<64, 128, 2, 2>;   // six accumulators (update backward)

struct Bump {
  size_t off = 0;
  size_t take(size_t bytes) {
    const size_t o = off;
    off += (bytes + 255) & ~size_t(255);
    return o;
  }
};

int ceil_div(int a, int b) { return (a + b - 1) / b; }

struct Split {
  int n, len;
};
// max_n: slots the partial-sum buffer holds for this launch
Split choose_split(int tokens, int tiles_total, int max_n) {
  // One split once the tiles alone occupy most of the 256 compute units: the partial sums then never exist.
  // Otherwise enough splits for one round of blocks, each over at least 1536 tokens: partial sums cost a write, a
  // read and (in the backward) a launch, which short splits do not earn back (measured at 36 to 72 tiles: 8.6 ->
  // 7.4 ms at config 2, 3.63 -> 3.41 ms at config 4 against a target of two rounds and 128 tokens).
  int ns = tiles_total >= 160 ? 1 : std::max(1, 256 / std::max(1, tiles_total));
  ns = std::min(std::min(ns, std::max(1, max_n)), std::max(1, tokens / 1536));
  int len = ceil_div(ceil_div(tokens, ns), 64) * 64;
  return Split{ceil_div(tokens, len), len};
}

// output tiles per matrix of the asynchronous-copy token reduction
int token_reduce_dma_tiles(int d, int dh) {
  const bool big = d % TS_NS::BM == 0 && dh % TS_NS::BM == 0;
  return big ? (d / TS_NS::BM) * (dh / TS_NS::BN)
             : std::max(ceil_div(dh, TS_SQ::BM) * ceil_div(d, TS_SQ::BN), ceil_div(d, TS_SQ::BM) * ceil_div(dh, TS_SQ::BN));
}

// One Newton-Schulz launch group: n matrices of one geometry, laid out one after the other.
struct NsBatch {
  int n, r, c;          // matrices, Newton-Schulz orientation [r, c] (r <= c)
  int mask, nb;         // the orthogonalised update of matrix z is written back transposed when bit (z / nb) of mask is set
  int first;            // index of its first matrix among all Newton-Schulz matrices (barrier lines)
  size_t xoff, sqoff;   // element offsets: [r, c]-shaped buffers (and the update in original orientation); [r, r]-shaped buffers
};

struct Plan {
  lact_desc_t d;
  std::vector<NsBatch> nsb;
  size_t sq_total = 0;    // elements of one [r, r]-shaped buffer over all batches
  std::vector<lact_step_t> steps;
  std::vector<lact_step_t> live;    // the steps that are executed: `steps` without the apply rows a later step overwrites
  std::vector<float> coeffs;
  MatGeom g;
  int nupd = 0, Tcap = 0, S = -1, esz = 2, nsz = 2, r = 0, c = 0, nblk = 1, lr_slots = 1, tiles = 1, nsplit_max = 1;
  bool muon = false, bf16 = true, momentum = false, state_in = false;
  size_t mat3 = 0;  // 3*b*elems
  // saved
  size_t s_n0, s_wf, s_wc, s_main, s_d, s_min, s_mbar, s_u, s_g16, s_norms, s_xb, s_ab, s_bb, saved_bytes;
  // Kept for the backward on the asynchronous-copy path: per update, six token-major arrays [b][T][dh] -- the three
  // lr-scaled hidden-side operands the backward's GEMMs read and the three rounded pre-activations they came from.
  // (The two unscaled operands of the forward's dw0 / dw2 reductions, which scale k instead, are read by the forward's
  // own token reduction only: they live in the call's scratch.)
  // 288 GB of HBM make keeping them cheaper than the three GEMMs that would recompute them.
  bool keep_pre = false;
  std::vector<size_t> s_pre;   // by update index
  std::vector<int> pre_T;
  // scratch
  size_t t_h[6], t_partial, t_lrpart, t_xf[2], t_xbtmp, t_ss, t_dot, t_mdot, t_gwhat[2], t_gwcur, t_gmcarry, t_gc,
      t_gxf[2], t_gxb[2], t_sg, t_gas, t_gn0, t_hs[3], t_partial_side, t_gwside[2], t_nssync, t_kl[2], t_ca, scratch_bytes;

  int build(const lact_desc_t* desc) {
    if (!desc) return fail("null descriptor");
    d = *desc;
    if (d.b <= 0 || d.d <= 0 || d.dh <= 0) return fail("b, d, dh must be positive");
    if (d.d % 8 || d.dh % 8) return fail("d and dh must be multiples of 8");
    if (d.act_dtype != LACT_BF16 && d.act_dtype != LACT_F32) return fail("act_dtype must be LACT_BF16 or LACT_F32");
    bf16 = d.act_dtype == LACT_BF16;
    esz = bf16 ? 2 : 4;
    const int al = bf16 ? 8 : 4;
    if (d.q_ld % al || d.k_ld % al || d.v_ld % al || d.o_ld % al || d.q_bs % al || d.k_bs % al || d.v_bs % al ||
        d.o_bs % al)
      return fail("row and batch strides must keep 16-byte alignment");
    if (d.q_ld < d.d || d.k_ld < d.d || d.v_ld < d.d || d.o_ld < d.d) return fail("row stride smaller than d");
    if (3LL * d.b > 65535) return fail("b too large (3*b must fit a grid dimension)");
    if (d.n_steps <= 0 || !d.steps) return fail("empty program");
    steps.assign(d.steps, d.steps + d.n_steps);
    S = d.ns_steps;
    muon = S >= 0;
    if (S > 0 && !d.ns_coeffs) return fail("ns_coeffs missing");
    if (S > 64) return fail("too many Newton-Schulz steps");
    if (S > 0) coeffs.assign(d.ns_coeffs, d.ns_coeffs + 3 * S);
    momentum = d.use_momentum != 0;
    state_in = d.momentum_state_in != 0;
    if (state_in && (!momentum || !d.forward_only))
      return fail("momentum_state_in needs use_momentum and forward_only (the carried state has no backward pass)");
    if (d.ns_mode < 0 || d.ns_mode > 2) return fail("ns_mode must be 0, 1 or 2");
    nsz = d.ns_mode == LACT_NS_FP32 ? 4 : 2;
    nupd = 0;
    Tcap = 0;
    for (const auto& s : steps) {
      if (s.kind != LACT_UPDATE && s.kind != LACT_APPLY) return fail("step kind must be LACT_UPDATE or LACT_APPLY");
      if (s.start < 0 || s.end <= s.start) return fail("empty or negative step range");
      if (s.kind == LACT_UPDATE) {
        if (s.end > d.kv_len) return fail("update range exceeds kv_len");
        ++nupd;
      } else {
        if (s.end > d.q_len) return fail("apply range exceeds q_len");
        if (s.out_start < 0 || s.out_start + (s.end - s.start) > d.out_len) return fail("apply output range exceeds out_len");
      }
      Tcap = std::max(Tcap, s.end - s.start);
    }
    // Output rows that a later apply step writes again are dead in the earlier one (the reference's slice
    // assignment lets the later write win, and no gradient reaches the overwritten values): every apply step is
    // cut down to the rows that survive, in the forward and in the backward alike.  What is left never writes a
    // row twice, so the apply steps may run in any order.
    live.clear();
    for (size_t i = 0; i < steps.size(); ++i) {
      const lact_step_t& a = steps[i];
      if (a.kind != LACT_APPLY) { live.push_back(a); continue; }
      std::vector<std::pair<int, int>> keep(1, std::make_pair(a.out_start, a.out_start + (a.end - a.start)));
      for (size_t j = i + 1; j < steps.size() && !keep.empty(); ++j) {
        const lact_step_t& b = steps[j];
        if (b.kind != LACT_APPLY) continue;
        const int b0 = b.out_start, b1 = b.out_start + (b.end - b.start);
        std::vector<std::pair<int, int>> next;
        for (auto& iv : keep) {
          if (b1 <= iv.first || iv.second <= b0) { next.push_back(iv); continue; }
          if (iv.first < b0) next.emplace_back(iv.first, b0);
          if (b1 < iv.second) next.emplace_back(b1, iv.second);
        }
        keep.swap(next);
      }
      for (auto& iv : keep) {
        lact_step_t c = a;
        c.start = a.start + (iv.first - a.out_start);
        c.end = c.start + (iv.second - iv.first);
        c.out_start = iv.first;
        live.push_back(c);
      }
    }
    g.d = d.d;
    g.dh = d.dh;
    g.nb = d.b;
    g.elems = (long long)d.d * d.dh;
    r = std::min(d.d, d.dh);
    c = std::max(d.d, d.dh);
    mat3 = (size_t)3 * d.b * g.elems;
    g.stacked = (muon && d.muon_stacked) ? 1 : 0;
    if (g.stacked && S == 0) return fail("muon_stacked needs at least one Newton-Schulz iteration");
    nsb.clear();
    if (!g.stacked) {
      nsb.push_back(NsBatch{3 * d.b, r, c, (g.tall(0) ? 1 : 0) | (g.tall(1) ? 2 : 0) | (g.tall(2) ? 4 : 0), d.b, 0, 0, 0});
      sq_total = (size_t)3 * d.b * r * r;
    } else {
      const int rs = std::min(2 * d.dh, d.d), cs = std::max(2 * d.dh, d.d);
      nsb.push_back(NsBatch{d.b, rs, cs, 2 * d.dh > d.d ? 1 : 0, d.b, 0, 0, 0});
      nsb.push_back(NsBatch{d.b, r, c, g.tall(1) ? 1 : 0, d.b, d.b, (size_t)2 * d.b * g.elems, (size_t)d.b * rs * rs});
      sq_total = (size_t)d.b * rs * rs + (size_t)d.b * r * r;
    }
    nblk = std::max(1, std::min(256, (int)((g.elems + 2047) / 2048)));
    lr_slots = ceil_div(d.dh, 128) * 4;   // (hidden tiles) x (wave columns) of the widest update-backward tiling
    tiles = ceil_div(d.dh, TSA::BM) * ceil_div(d.d, TSA::BN);
    tiles = std::max(tiles, ceil_div(d.d, TSA::BM) * ceil_div(d.dh, TSA::BN));
    // partial-sum slots: the larger split count of the two token-reduction kernels at the longest chunk (the
    // count grows with the tokens) + the slot of a ragged tail
    nsplit_max = std::max(choose_split(Tcap, tiles * 3 * d.b, 16).n, choose_split(Tcap, token_reduce_dma_tiles(d.d, d.dh) * 3 * d.b, 16).n) + 1;

    Bump sv;
    s_n0 = sv.take((size_t)3 * d.b * g.maxrows() * 4);
    s_wf = sv.take((size_t)(nupd + 1) * mat3 * 4);
    s_wc = bf16 ? sv.take((size_t)(nupd + 1) * mat3 * 2) : s_wf;
    s_main = d.prenorm ? sv.take((size_t)nupd * mat3 * 4) : 0;
    s_d = sv.take((size_t)nupd * mat3 * 4);
    s_min = state_in ? sv.take(mat3 * 4) : 0;
    s_mbar = sv.take((size_t)std::max(1, nupd) * d.b * 4);
    s_u = muon ? sv.take((size_t)nupd * mat3 * 4) : 0;
    s_g16 = muon ? sv.take((size_t)nupd * mat3 * nsz) : 0;
    s_norms = sv.take((size_t)std::max(1, nupd) * 3 * d.b * 4);
    s_xb = muon ? sv.take((size_t)nupd * std::max(1, S) * mat3 * nsz) : 0;
    const size_t sq3 = sq_total;
    s_ab = muon ? sv.take((size_t)nupd * std::max(1, S) * sq3 * nsz) : 0;
    s_bb = muon ? sv.take((size_t)nupd * std::max(1, S) * sq3 * nsz) : 0;
    // Keep the update's rounded pre-activations and lr-scaled operands for the backward (three GEMM phases there
    // instead of six), or let the backward recompute them?  Recomputing costs K = d of matrix work per tile and saves
    // five token-major arrays of stores in the forward: at d <= 128 (two K-steps) recomputing wins (d = 128, dh = 256,
    // 32760 tokens: 3.61 against 3.70 ms per step), at d = 384 keeping does (1.298 against 1.316 ms; 7.38 against 7.47).
    keep_pre = bf16 && d.d % 64 == 0 && d.dh % 64 == 0 && !d.forward_only && (g_keep_pre < 0 ? d.d > 128 : g_keep_pre != 0);
    s_pre.clear(); pre_T.clear();
    if (keep_pre)
      for (const auto& st : steps)
        if (st.kind == LACT_UPDATE) {
          pre_T.push_back(st.end - st.start);
          s_pre.push_back(sv.take((size_t)6 * d.b * (st.end - st.start) * d.dh * esz));
        }
    saved_bytes = sv.off + 256;

    Bump sc;
    for (int i = 0; i < 6; ++i) t_h[i] = sc.take((size_t)d.b * Tcap * d.dh * esz);
    t_partial = sc.take((size_t)nsplit_max * mat3 * 4);
    t_lrpart = sc.take((size_t)std::max(1, nupd) * 3 * lr_slots * d.b * Tcap * 4);   // one slot per update: reduced by one launch at the end
    for (int i = 0; i < 2; ++i) t_xf[i] = sc.take(mat3 * 4);
    t_xbtmp = sc.take(mat3 * nsz);
    t_ss = sc.take((size_t)3 * d.b * nblk * 4);
    t_dot = sc.take((size_t)3 * d.b * std::max(nblk, 32) * 4);   // partial dots: per chunk of a matrix, or per block of the fused kernel
    t_mdot = sc.take((size_t)std::max(1, nupd) * 3 * d.b * std::max(nblk, 256) * 4);   // one slot per update: the momentum gradients are written at the end
    for (int i = 0; i < 2; ++i) t_gwhat[i] = sc.take(mat3 * 4);
    t_gwcur = sc.take(mat3 * 4);
    t_gmcarry = sc.take(mat3 * 4);
    t_gc = sc.take(mat3 * esz);
    for (int i = 0; i < 2; ++i) t_gxf[i] = sc.take(mat3 * 4);
    for (int i = 0; i < 2; ++i) t_gxb[i] = sc.take(mat3 * nsz);
    t_sg = sc.take(sq3 * nsz);
    t_gas = sc.take(sq3 * nsz);
    t_gn0 = sc.take((size_t)3 * d.b * g.maxrows() * 4);
    // the apply steps' own buffers (they run beside the update chain)
    for (int i = 0; i < 3; ++i) t_hs[i] = sc.take((size_t)d.b * Tcap * d.dh * esz);
    t_partial_side = sc.take((size_t)nsplit_max * mat3 * 4);
    for (int i = 0; i < 2; ++i) t_gwside[i] = sc.take(mat3 * 4);
    t_nssync = sc.take(((size_t)3 * d.b * 32 + 32) * 4);   // per-matrix barrier lines of the fused Newton-Schulz kernel + error word
    for (int i = 0; i < 2; ++i) t_kl[i] = sc.take((size_t)d.b * Tcap * d.d * esz);   // k * lr0, k * lr2 of the current update
    t_ca = muon ? sc.take(sq3 * nsz) : 0;                   // c * A of the current Newton-Schulz iteration
    scratch_bytes = sc.off + 256;
    return 0;
  }
};

inline char* align256(void* p) { return reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~uintptr_t(255)); }
inline const char* align256(const void* p) {
  return reinterpret_cast<const char*>((reinterpret_cast<uintptr_t>(p) + 255) & ~uintptr_t(255));
}

template <typename T, bool B_KC, int NT, int EPI>
const char* row_gemm_name() {
  static const std::string n = std::string("k_row_gemm<") + tname<T>() + (B_KC ? ",Bkc," : ",Bks,") + std::to_string(NT) +
                               (EPI == EPI_STORE ? ",store>" : (EPI == EPI_AXPBY ? ",axpby>" : ",axpby_dual>"));
  return n.c_str();
}
template <class TS, int NT, int EPI, bool B_KS>
void launch_row_gemm_dma(const char* site, const RowGemmDmaParams<NT>& q, int batch, hipStream_t s) {
  constexpr int STAGES = row_stages<TS>();
  constexpr int SMEM = cmax(DmaSmem<TS, 1, STAGES>::BYTES, StageTile<TS, 4>::BYTES);
  LACT_BIG_LDS((k_row_gemm_dma<TS, NT, EPI, B_KS>), SMEM);
  static const std::string name = std::string("k_row_gemm_dma<") + std::to_string(TS::BM) + "x" + std::to_string(TS::BN) + "," +
                                  std::to_string(NT) + (EPI == EPI_STORE ? ",store" : (EPI == EPI_AXPBY ? ",axpby" : ",axpby_dual")) +
                                  (B_KS ? ",Bks>" : ",Bkc>");
  RowGemmDmaParams<NT> qq = q;
  qq.map = make_tile_map(ceil_div(q.g.M, TS::BM), ceil_div(q.g.N, TS::BN), batch);
  double ksum = 0;
  for (int t = 0; t < NT; ++t) ksum += q.g.t[t].K;
  LACT_LAUNCH_SMEM(name.c_str(), site, 2.0 * q.g.M * q.g.N * ksum * batch, (k_row_gemm_dma<TS, NT, EPI, B_KS>), dim3(qq.map.grid()),
                   dim3(DMA_THREADS), SMEM, s, qq);
}
// bf16 with every K a multiple of 64: asynchronous-copy kernels; anything else: the generic tile loop
template <typename T, bool B_KC, int NT, int EPI>
void launch_row_gemm(const char* site, const RowGemmParams<NT>& p, int batch, hipStream_t s, bool token_rows = false) {
  if constexpr (std::is_same<T, uint16_t>::value) {
    bool ok = p.N % 8 == 0;
    for (int t = 0; t < NT; ++t) ok = ok && p.t[t].K % 64 == 0;
    if (ok) {
      RowGemmDmaParams<NT> q;
      q.g = p;
      q.out_ct = nullptr;
      if (token_rows) {
        // 256 x 128 tiles copy a third fewer operand bytes per FLOP than 128 x 128 ones, but a launch whose blocks fill
        // the last round of compute units only partly wastes more than that: pick by the fuller last round
        static const int cus = [] { int dev = 0, n = 0; (void)hipGetDevice(&dev); return hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256; }();
        auto fill = [&](int bm) { const long long blocks = (long long)ceil_div(p.M, bm) * ceil_div(p.N, 128) * batch; return (double)blocks / ((double)((blocks + cus - 1) / cus) * cus); };
        // (measured at 384 blocks on 256 units: one-term GEMM 27.0 -> 24.5 us with the small tile, two-term GEMM with
        // K-strided weights 34 -> 36 us: only the one-term case switches)
        if (NT == 1 && fill(256) < 0.8 && fill(128) > fill(256) + 0.1) launch_row_gemm_dma<TS_SQ, NT, EPI, !B_KC>(site, q, batch, s);
        else launch_row_gemm_dma<TS_ROW, NT, EPI, !B_KC>(site, q, batch, s);
      }
      else if (p.M % TS_NS::BM == 0 && p.N % TS_NS::BN == 0) launch_row_gemm_dma<TS_NS, NT, EPI, !B_KC>(site, q, batch, s);
      else launch_row_gemm_dma<TS_SQ, NT, EPI, !B_KC>(site, q, batch, s);
      return;
    }
  }
  dim3 grid(ceil_div(p.M, TSA::BM), ceil_div(p.N, TSA::BN), batch);
  double ksum = 0;
  for (int t = 0; t < NT; ++t) ksum += p.t[t].K;
  LACT_LAUNCH((row_gemm_name<T, B_KC, NT, EPI>()), site, 2.0 * p.M * p.N * ksum * batch,
              (k_row_gemm<T, TSA, B_KC, NT, EPI>), grid, dim3(TSA::THREADS), s, p);
}

template <int NT>
RowGemmParams<NT> row_params() {
  RowGemmParams<NT> p;
  memset(&p, 0, sizeof(p));
  p.alpha = 1.f;
  return p;
}

inline void set_term(RowGemmTerm& t, const void* A, int lda, long long bsA, const void* B, int ldb, long long bsB, int K) {
  t.A = A; t.lda = lda; t.bsA = bsA; t.B = B; t.ldb = ldb; t.bsB = bsB; t.K = K;
}
inline void set_tr_term(TokenReduceTerm& t, const void* A, int lda, long long bsA, const void* B, int ldb, long long bsB) {
  t.A = A; t.lda = lda; t.bsA = bsA; t.B = B; t.ldb = ldb; t.bsB = bsB;
}

// One Newton-Schulz iteration on n matrices held as [r, c] (always bf16 MFMA, fp32 iterate):
//   A = X X^T;  B = b A + c A A;  X' = a X + B X        (ttt_operation.py:59-62)
struct NsIter {
  int n, r, c, nb_for_mask, mask, plain;
  float ca, cb, cc;
  const float* xf_in; const void* xb_in;           // X: fp32 iterate and its copy in the GEMM type
  void* ab; void* bb;                              // A and B of this iteration (GEMM type)
  void* cab;                                       // c * A (GEMM type): the left operand of (c * A) @ A, a tensor of its own in the reference
  float* xf_out; void* xb_out; float* u_out;       // X': fp32, GEMM type, and fp32 in the original orientation (each nullable)
};
// TN: GEMM operand type of the iteration (bf16 as in the reference, or fp32 for the exact mode)
template <typename TN>
void ns_iteration(const NsIter& I, hipStream_t s) {
  const long long xe = (long long)I.r * I.c, se = (long long)I.r * I.r;
  {
    auto p = row_params<1>();
    set_term(p.t[0], I.xb_in, I.c, xe, I.xb_in, I.c, xe, I.c);
    p.M = I.r; p.N = I.r; p.out = I.ab; p.ldo = I.r; p.bso = se;
    p.out2 = I.cab; p.alpha2 = I.cc;
    launch_row_gemm<TN, true, 1, EPI_STORE>("ns_gram", p, I.n, s);
  }
  {   // B = b * A + (c * A) @ A, ttt_operation.py:60
    auto p = row_params<1>();
    set_term(p.t[0], I.cab, I.r, se, I.ab, I.r, se, I.r);
    p.M = I.r; p.N = I.r; p.out = I.bb; p.ldo = I.r; p.bso = se;
    p.aux = I.ab; p.ldaux = I.r; p.bsaux = se; p.alpha = 1.f; p.beta = I.cb;
    launch_row_gemm<TN, true, 1, EPI_AXPBY>("ns_poly", p, I.n, s);
  }
  {
    auto p = row_params<1>();
    set_term(p.t[0], I.bb, I.r, se, I.xb_in, I.c, xe, I.r);
    p.M = I.r; p.N = I.c; p.ldo = I.c; p.bso = xe;
    p.aux = I.xf_in; p.ldaux = I.c; p.bsaux = xe; p.alpha = 1.f; p.beta = I.ca;
    p.round_out_bf16 = I.plain;
    p.out = I.xf_out; p.out_c = I.xb_out; p.out_t = I.u_out;
    p.transpose_mask = I.mask; p.nb = I.nb_for_mask;
    launch_row_gemm<TN, false, 1, EPI_AXPBY_F32_DUAL>("ns_next", p, I.n, s);
  }
}

template <typename T, typename TN>
struct Runner {
  const Plan& P;
  hipStream_t s;
  char* sv;   // saved
  char* sc;   // scratch
  const lact_desc_t& d;
  hipStream_t s_main, s_side;   // caller's stream; stream of the apply steps (= s_main when overlap is off)
  hipStream_t s_tail;           // stream of dk, dv and the learning-rate gradients (= s_main when overlap is off)
  SideCtx* side = nullptr;
  const size_t* hsel;           // token-major intermediates of the chain being enqueued
  size_t partial_sel;
  Runner(const Plan& p, void* saved, void* scratch, hipStream_t st)
      : P(p), s(st), sv(align256(saved)), sc(align256(scratch)), d(p.d), s_main(st), s_side(st), s_tail(st), hsel(p.t_h), partial_sel(p.t_partial) {
    side = side_ctx();
    if (side && g_overlap) { s_side = side->stream; s_tail = side->tail; }
  }
  // ---- fused Newton-Schulz: launches of at most 256 resident blocks
  static bool tiles_fit(int r, int c, int bm, int bn) {
    return r % bm == 0 && r % bn == 0 && c % bn == 0 && (r / bm) * (c / bn) <= 32;
  }
  // Tile of the fused kernel for a batch: 0 = 192 x 192, 1 = 128 x 128, 2 = 128 x 64, 3 = 128 x 96, -1 = none fits.
  // 192 x 192 when the matrices fill at least half the chip with it, else 128 x 128 (more, smaller blocks), and
  // 128 x 64 or 128 x 96 when even those leave most of the chip idle -- as long as the groups dealt to one XCD (a
  // matrix's blocks share an XCD) still find a compute unit each there.
  static int ns_fused_tile(const NsBatch& B) {
    const bool f192 = tiles_fit(B.r, B.c, 192, 192), f128 = tiles_fit(B.r, B.c, 128, 128), f64 = tiles_fit(B.r, B.c, 128, 64);
    const bool f96 = tiles_fit(B.r, B.c, 128, 96);
    if (f192 && (!f128 || B.n * (B.r / 192) * (B.c / 192) >= 128)) return 0;
    const int per_xcd = (B.n + 7) / 8;
    const bool sparse128 = !f128 || B.n * (B.r / 128) * (B.c / 128) < 128;
    if (f64) {
      const int nbm64 = (B.r / 128) * (B.c / 64);
      if (per_xcd * nbm64 <= 32 && sparse128) return 2;
    }
    if (f96) {
      const int nbm96 = (B.r / 128) * (B.c / 96);
      if (per_xcd * nbm96 <= 32 && sparse128) return 3;
    }
    if (f128) return 1;
    return f192 ? 0 : -1;
  }
  static int ns_fused_nbm(const NsBatch& B) {   // blocks per matrix of the fused kernel
    switch (ns_fused_tile(B)) {
      case 0: return (B.r / 192) * (B.c / 192);
      case 1: return (B.r / 128) * (B.c / 128);
      case 2: return (B.r / 128) * (B.c / 64);
      case 3: return (B.r / 128) * (B.c / 96);
      default: return 0;
    }
  }
  // The fused kernel's groups must be resident as a whole, one block per compute unit, on a device that deals its
  // workgroups to 8 dies of 32 compute units: anything else (a partitioned or smaller device) takes the unfused launches.
  bool ns_fusable(const NsBatch& B) const {
    if (!side || !kNsBf16 || P.S < 1 || P.S > NS_FUSED_MAX_STEPS) return false;
    if (side->cus < 256) return false;
    return ns_fused_tile(B) >= 0;
  }
  bool ns_fused_ok(const NsBatch& B) const { return g_fused_ns && ns_fusable(B); }
  // The unfused launches of a batch the fused kernel could take sum the dot product of the normalisation's backward
  // over the fused kernel's tiles, in its order: switching LACT_OPT_FUSED_NEWTON_SCHULZ then changes no bit.
  bool ns_dot_by_tiles() const { return P.muon && P.nsb.size() == 1 && ns_fusable(P.nsb[0]); }
  template <class TS>
  void launch_ns_dot_tiles_ts(const NsTileDotParams& q, const NsBatch& B) {
    LACT_LAUNCH("k_ns_bwd_dot_tiles", "k_ns_bwd_dot", 0.0, (k_ns_bwd_dot_tiles<TS>), dim3((B.r / TS::BM) * (B.c / TS::BN), B.n), dim3(DMA_THREADS), s, q);
  }
  void launch_ns_dot_tiles(const NsTileDotParams& q, const NsBatch& B) {
    switch (ns_fused_tile(B)) {
      case 0: launch_ns_dot_tiles_ts<TS_NS>(q, B); break;
      case 1: launch_ns_dot_tiles_ts<TS_SQ>(q, B); break;
      case 2: launch_ns_dot_tiles_ts<TS_BWD>(q, B); break;
      case 3: launch_ns_dot_tiles_ts<TS_N96>(q, B); break;
      default: break;
    }
  }
  // every batch runs fused (and at least one iteration): the Frobenius normalisation is the fused kernel's first stage
  bool ns_all_fused() const {
    if (!P.muon || P.nsb.empty()) return false;
    for (auto& B : P.nsb)
      if (!ns_fused_ok(B)) return false;
    return true;
  }
  bool ns_fused_any() const {
    for (auto& B : P.nsb)
      if (ns_fused_ok(B)) return true;
    return false;
  }
  unsigned* ns_error_word() const { return scr<unsigned>(P.t_nssync) + (size_t)P.g.ns_count() * 32; }
  // barrier lines and error word start at zero: once per Newton-Schulz phase, by the kernel in front of its batches
  ClearWords ns_clear() const {
    ClearWords c;
    c.ptr = nullptr; c.n = 0;
    if (P.muon && ns_fused_any()) { c.ptr = scr<unsigned>(P.t_nssync); c.n = P.g.ns_count() * 32 + 32; }
    return c;
  }
  template <class TS, bool BWD>
  void launch_ns_fused_ts(NsFusedParams p, const NsBatch& B) {
    constexpr int SM = cmax(DmaSmem<TS, 1, row_stages<TS>()>::BYTES, StageTile<TS, 4>::BYTES);
    LACT_BIG_LDS((k_ns_fused<TS, BWD>), SM);
    const int nbm = (B.r / TS::BM) * (B.c / TS::BN);
    const int per = (256 / nbm) / 8 * 8;
    unsigned* sync = scr<unsigned>(P.t_nssync) + (size_t)B.first * 32;
    p.r = B.r; p.c = B.c; p.S = P.S; p.nb = B.nb; p.mask = B.mask;
    for (int i = 0; i < 3 * P.S; ++i) p.coeffs[i] = P.coeffs[i];
    p.error = ns_error_word();
    p.sticky = side->sticky;
    p.spin_limit = g_ns_spin_limit;
    const double terms = BWD ? 6.0 : 3.0;
    static const std::string name = std::string("k_ns_fused<") + std::to_string(TS::BM) + "x" + std::to_string(TS::BN) + (BWD ? ",bwd>" : ",fwd>");
    for (int z0 = 0; z0 < B.n; z0 += per) {
      p.z0 = z0; p.n = std::min(per, B.n - z0); p.sync = sync + (size_t)z0 * 32;
      const int grid = 8 * ((p.n + 7) / 8) * nbm;
      side->order_fused_launch(s);
      LACT_LAUNCH_SMEM(name.c_str(), BWD ? "ns_bwd" : "ns_fwd", terms * 2.0 * B.r * B.r * B.c * P.S * p.n,
                       (k_ns_fused<TS, BWD>), dim3(grid), dim3(DMA_THREADS), SM, s, p);
    }
  }
  template <bool BWD>
  void launch_ns_fused(const NsFusedParams& p, const NsBatch& B) {
    switch (ns_fused_tile(B)) {
      case 0: launch_ns_fused_ts<TS_NS, BWD>(p, B); break;
      case 1: launch_ns_fused_ts<TS_SQ, BWD>(p, B); break;
      case 2: launch_ns_fused_ts<TS_BWD, BWD>(p, B); break;
      case 3: launch_ns_fused_ts<TS_N96, BWD>(p, B); break;
      default: break;
    }
  }
  // `waiter` waits for everything enqueued so far on `on`
  void wait_for(hipStream_t waiter, hipStream_t on) {
    if (waiter == on || !side) return;
    hipEvent_t e = side->event();
    (void)hipEventRecord(e, on);
    (void)hipStreamWaitEvent(waiter, e, 0);
  }
  // enqueue on the side chain (its stream and buffers) while this object lives
  struct OnSide {
    Runner& r;
    explicit OnSide(Runner& rr) : r(rr) { r.s = r.s_side; r.hsel = r.P.t_hs; r.partial_sel = r.P.t_partial_side; }
    ~OnSide() { r.s = r.s_main; r.hsel = r.P.t_h; r.partial_sel = r.P.t_partial; }
  };

  float* n0() const { return reinterpret_cast<float*>(sv + P.s_n0); }
  float* wf(int ver) const { return reinterpret_cast<float*>(sv + P.s_wf) + (size_t)ver * P.mat3; }
  T* wc(int ver) const { return reinterpret_cast<T*>(sv + P.s_wc) + (size_t)ver * P.mat3; }
  T* wc(int ver, int j) const { return wc(ver) + (size_t)j * d.b * P.g.elems; }
  // accumulator after `u` updates (pre-norm); main(0) is the initial weight
  float* main_(int u) const { return u == 0 ? wf(0) : reinterpret_cast<float*>(sv + P.s_main) + (size_t)(u - 1) * P.mat3; }
  float* dsave(int u) const { return reinterpret_cast<float*>(sv + P.s_d) + (size_t)u * P.mat3; }
  // momentum state that update `u` starts from: the previous update's, or the one the caller carried in
  bool has_prev(int u) const { return P.momentum && (u > 0 || P.state_in); }
  const float* mprev(int u) const { return !has_prev(u) ? nullptr : u > 0 ? dsave(u - 1) : reinterpret_cast<const float*>(sv + P.s_min); }
  float* mbar(int u) const { return reinterpret_cast<float*>(sv + P.s_mbar) + (size_t)u * d.b; }
  float* usave(int u) const { return reinterpret_cast<float*>(sv + P.s_u) + (size_t)u * P.mat3; }
  TN* g16(int u) const { return reinterpret_cast<TN*>(sv + P.s_g16) + (size_t)u * P.mat3; }
  float* norms(int u) const { return reinterpret_cast<float*>(sv + P.s_norms) + (size_t)u * 3 * d.b; }
  TN* xb(int u, int it) const { return reinterpret_cast<TN*>(sv + P.s_xb) + ((size_t)u * std::max(1, P.S) + it) * P.mat3; }
  size_t sq3() const { return P.sq_total; }
  TN* ab(int u, int it) const { return reinterpret_cast<TN*>(sv + P.s_ab) + ((size_t)u * std::max(1, P.S) + it) * sq3(); }
  TN* bb(int u, int it) const { return reinterpret_cast<TN*>(sv + P.s_bb) + ((size_t)u * std::max(1, P.S) + it) * sq3(); }
  T* h(int i) const { return reinterpret_cast<T*>(sc + hsel[i]); }
  // kept array i (0..2: lr-scaled operands, 3..5: pre-activations) of update u; batch stride pre_bs(u)
  T* pre(int u, int i) const { return reinterpret_cast<T*>(sv + P.s_pre[u]) + (size_t)i * d.b * P.pre_T[u] * d.dh; }
  long long pre_bs(int u) const { return (long long)P.pre_T[u] * d.dh; }
  static constexpr bool kBf16 = std::is_same<T, uint16_t>::value;
  static constexpr bool kNsBf16 = std::is_same<TN, uint16_t>::value;

  // the hidden-stage kernels with asynchronous copies need bf16 and whole 64-element K-steps
  bool dma_hidden() const { return kBf16 && d.d % 64 == 0; }
  // row-partial slots the update-backward hidden kernel in use writes: (hidden tiles) x (wave columns)
  int lr_parts() const {
    if (!dma_hidden()) return ceil_div(d.dh, TSB::BN) * TSB::WAVES_N;
    if (P.keep_pre) return ceil_div(d.dh, TS_SQ::BN) * TS_SQ::WAVES_N;
    return ceil_div(d.dh, TS_BWD::BN) * TS_BWD::WAVES_N;
  }
  void launch_hidden(int which, const HiddenParams& hp, int ver, int T_) const {
    const double f = (double)T_ * d.d * d.dh * d.b;
    if (dma_hidden()) {
      if constexpr (kBf16) {
      HiddenDmaParams q;
      q.h = hp;
      (void)ver;
      constexpr int SM3 = DmaSmem<TS_SQ, 2, 3>::BYTES;   // the epilogues stage at most three bf16 tiles, inside the ring
      constexpr int SM6 = cmax(DmaSmem<TS_BWD, 2, 3>::BYTES, 6 * StageTile<TS_BWD, 2>::BYTES);
      const TileMap m3 = make_tile_map(ceil_div(T_, TS_SQ::BM), ceil_div(d.dh, TS_SQ::BN), d.b);
      const TileMap m6 = make_tile_map(ceil_div(T_, TS_BWD::BM), ceil_div(d.dh, TS_BWD::BN), d.b);
      q.map = which == 3 ? m6 : m3;
      dim3 g3(m3.grid()), g6(m6.grid());
      LACT_BIG_LDS(k_apply_hidden_dma<TS_SQ>, SM3);
      LACT_BIG_LDS(k_update_hidden_dma<TS_SQ>, SM3);
      LACT_BIG_LDS(k_apply_bwd_hidden_dma<TS_SQ>, SM3);
      LACT_BIG_LDS(k_update_bwd_hidden_dma<TS_BWD>, SM6);
      LACT_BIG_LDS(k_update_bwd_hidden_kept_dma<TS_SQ>, SM3);
      if (which <= 2 && ((g_persist >> which) & 1) && side && side->cus > 0) {
        HiddenPersistParams hq;
        hq.h = hp; hq.map = m3;
        const dim3 gp(persist_grid(m3.grid(), side->cus));
        LACT_BIG_LDS(k_hidden_persist<ApplyHiddenPolicy>, PersistLds<ApplyHiddenPolicy>::BYTES);
        LACT_BIG_LDS(k_hidden_persist<UpdateHiddenPolicy>, PersistLds<UpdateHiddenPolicy>::BYTES);
        LACT_BIG_LDS(k_hidden_persist<ApplyBwdHiddenPolicy>, PersistLds<ApplyBwdHiddenPolicy>::BYTES);
        if (which == 0) LACT_LAUNCH_SMEM("k_hidden_persist<apply>", "apply_hidden", 4.0 * f, (k_hidden_persist<ApplyHiddenPolicy>), gp, dim3(DMA_THREADS), PersistLds<ApplyHiddenPolicy>::BYTES, s, hq);
        if (which == 1) LACT_LAUNCH_SMEM("k_hidden_persist<update>", "update_hidden", 6.0 * f, (k_hidden_persist<UpdateHiddenPolicy>), gp, dim3(DMA_THREADS), PersistLds<UpdateHiddenPolicy>::BYTES, s, hq);
        if (which == 2) LACT_LAUNCH_SMEM("k_hidden_persist<apply_bwd>", "apply_bwd_hidden", 6.0 * f, (k_hidden_persist<ApplyBwdHiddenPolicy>), gp, dim3(DMA_THREADS), PersistLds<ApplyBwdHiddenPolicy>::BYTES, s, hq);
        return;
      }
      if (which == 0) LACT_LAUNCH_SMEM("k_apply_hidden_dma", "apply_hidden", 4.0 * f, (k_apply_hidden_dma<TS_SQ>), g3, dim3(DMA_THREADS), SM3, s, q);
      if (which == 1) LACT_LAUNCH_SMEM("k_update_hidden_dma", "update_hidden", 6.0 * f, (k_update_hidden_dma<TS_SQ>), g3, dim3(DMA_THREADS), SM3, s, q);
      if (which == 2) LACT_LAUNCH_SMEM("k_apply_bwd_hidden_dma", "apply_bwd_hidden", 6.0 * f, (k_apply_bwd_hidden_dma<TS_SQ>), g3, dim3(DMA_THREADS), SM3, s, q);
      if (which == 3) LACT_LAUNCH_SMEM("k_update_bwd_hidden_dma", "update_bwd_hidden", 12.0 * f, (k_update_bwd_hidden_dma<TS_BWD>), g6, dim3(DMA_THREADS), SM6, s, q);
      if (which == 4) LACT_LAUNCH_SMEM("k_update_bwd_hidden_kept_dma", "update_bwd_hidden", 6.0 * f, (k_update_bwd_hidden_kept_dma<TS_SQ>), g3, dim3(DMA_THREADS), SM3, s, q);
      }
    } else {
      dim3 ga(ceil_div(T_, TSA::BM), ceil_div(d.dh, TSA::BN), d.b), gb(ceil_div(T_, TSB::BM), ceil_div(d.dh, TSB::BN), d.b);
      if (which == 0) LACT_LAUNCH("k_apply_hidden", "apply_hidden", 4.0 * f, (k_apply_hidden<T, TSA>), ga, dim3(TSA::THREADS), s, hp);
      if (which == 1) LACT_LAUNCH("k_update_hidden", "update_hidden", 6.0 * f, (k_update_hidden<T, TSA>), ga, dim3(TSA::THREADS), s, hp);
      if (which == 2) LACT_LAUNCH("k_apply_bwd_hidden", "apply_bwd_hidden", 6.0 * f, (k_apply_bwd_hidden<T, TSA>), ga, dim3(TSA::THREADS), s, hp);
      if (which == 3) LACT_LAUNCH("k_update_bwd_hidden", "update_bwd_hidden", 12.0 * f, (k_update_bwd_hidden<T, TSB>), gb, dim3(TSB::THREADS), s, hp);
    }
  }
  template <typename U> U* scr(size_t off) const { return reinterpret_cast<U*>(sc + off); }

  long long hbs() const { return (long long)P.Tcap * d.dh; }

  HiddenParams hidden_params(int T_, const void* X, int ldx, long long bsx, const void* Y, int ldy, long long bsy, int ver) const {
    HiddenParams p;
    memset(&p, 0, sizeof(p));
    p.T = T_; p.d = d.d; p.dh = d.dh;
    p.X = X; p.ldx = ldx; p.bsx = bsx;
    p.Y = Y; p.ldy = ldy; p.bsy = bsy;
    p.W0 = wc(ver, 0); p.W1 = wc(ver, 1); p.W2 = wc(ver, 2); p.bsw = P.g.elems;
    p.bso = hbs();
    p.Tcap = P.Tcap;
    return p;
  }

  // The three token-reduction GEMMs of a step.  Returns the number of partial-sum slots written to the scratch
  // buffer (the caller reduces them), or 0 when the result went straight to `add_out` = coeff*add_in + sum.
  // bf16, 64 tokens or more: the asynchronous-copy kernel (straight to add_out when one split covers them; a token
  // count that is not a multiple of 64 ends inside the last K-step, whose surplus rows the loader clears).
  // `prep` (forward update only): d_out / g16 / ss_part / m_prev / mbar of the momentum step; when the whole
  // reduction is one split of the asynchronous-copy kernel, its epilogue does that step and -1 is returned.
  struct PrepFold {
    float* d_out; const float* m_prev; const float* mbar; uint16_t* g16; float* ss_part;
    bool skip_d;
    float* m_ext[3];
    ClearWords clear;
  };
  // `rows`: two token-row GEMMs (four and two terms, dk and dv of an update's backward) that may ride in the same
  // launch as the asynchronous-copy reduction; `done` tells the caller whether they did.
  struct RowCompanions {
    RowGemmParams<4> r4;
    RowGemmParams<2> r2;
    bool done = false;
  };
  int token_reduce(const char* site, const TokenReduceJob (&jobs)[3], int tokens, float* add_out = nullptr,
                   const float* add_in = nullptr, float coeff = 0.f, const PrepFold* prep = nullptr,
                   RowCompanions* rows = nullptr) const {
    TokenReduceParams p;
    memset(&p, 0, sizeof(p));
    for (int i = 0; i < 3; ++i) p.job[i] = jobs[i];
    p.nb = d.b; p.mat_elems = P.g.elems;
    float* partial = scr<float>(partial_sel);
    const dim3 flat((unsigned)((P.mat3 / 4 + 255) / 256));
    int main_tokens = 0, slots = 0;
    bool direct = false;
    if constexpr (kBf16) {
      if (tokens >= 64 && d.d % 8 == 0 && d.dh % 8 == 0) main_tokens = tokens;   // a ragged end is handled inside the last K-step
      if (main_tokens > 0) {
        const bool big = d.d % TS_NS::BM == 0 && d.dh % TS_NS::BM == 0;
        const int tiles = token_reduce_dma_tiles(d.d, d.dh);
        const Split sp = choose_split(main_tokens, tiles * 3 * d.b, P.nsplit_max - 1);
        TokenReduceDmaParams pd;
        static_cast<TokenReduceParams&>(pd) = p;
        pd.tokens = main_tokens; pd.split_len = sp.len; pd.partial = partial;
        pd.map = make_tile_map(sp.n, tiles, 3 * d.b);
        dim3 g(pd.map.grid());
        const double fl = 6.0 * main_tokens * d.d * d.dh * d.b * jobs[0].nterms;
        direct = add_out && sp.n == 1;
        const bool folded = prep && sp.n == 1 && main_tokens == tokens;
        if (folded) {
          pd.prep_d_out = prep->d_out; pd.prep_m_prev = prep->m_prev; pd.prep_mbar = prep->mbar; pd.prep_skip_d = prep->skip_d ? 1 : 0;
          pd.prep_g16 = prep->g16; pd.prep_ss_part = prep->ss_part; pd.prep_clear = prep->clear;
          for (int j = 0; j < 3; ++j) pd.prep_m_ext[j] = prep->m_ext[j];
        } else if (direct) { pd.add_out = add_out; pd.add_in = coeff != 0.f ? add_in : nullptr; pd.coeff = coeff; }
        else slots = sp.n;
        bool with_rows = rows != nullptr && rows->r4.N % 8 == 0 && rows->r2.N % 8 == 0;
        if (with_rows) {
          for (int t = 0; t < 4; ++t) with_rows = with_rows && rows->r4.t[t].K % 64 == 0;
          for (int t = 0; t < 2; ++t) with_rows = with_rows && rows->r2.t[t].K % 64 == 0;
        }
        if (with_rows) {
          TokenReduceRowsParams q;
          q.tr = pd;
          q.r4.g = rows->r4; q.r4.out_ct = nullptr;
          q.r4.map = make_tile_map(ceil_div(rows->r4.M, TS_ROW::BM), ceil_div(rows->r4.N, TS_ROW::BN), d.b);
          q.r2.g = rows->r2; q.r2.out_ct = nullptr;
          q.r2.map = make_tile_map(ceil_div(rows->r2.M, TS_ROW::BM), ceil_div(rows->r2.N, TS_ROW::BN), d.b);
          q.ntr = pd.map.grid(); q.n4 = q.r4.map.grid();
          const dim3 gr(q.ntr + q.n4 + q.r2.map.grid());
          double frows = 0;
          for (int t = 0; t < 4; ++t) frows += 2.0 * rows->r4.M * rows->r4.N * rows->r4.t[t].K * d.b;
          for (int t = 0; t < 2; ++t) frows += 2.0 * rows->r2.M * rows->r2.N * rows->r2.t[t].K * d.b;
          constexpr int SMR = cmax(DmaSmem<TS_ROW, 1, row_stages<TS_ROW>()>::BYTES, StageTile<TS_ROW, 4>::BYTES);
          if (big) {
            constexpr int SM = cmax(SMR, cmax(DmaSmem<TS_NS, 1, row_stages<TS_NS>()>::BYTES, StageTile<TS_NS, 4>::BYTES));
            LACT_BIG_LDS(k_token_reduce_rows_dma<TS_NS>, SM);
            LACT_LAUNCH_SMEM("k_token_reduce_rows_dma<192x192>", site, fl + frows, (k_token_reduce_rows_dma<TS_NS>), gr, dim3(DMA_THREADS), SM, s, q);
          } else {
            constexpr int SM = cmax(SMR, cmax(DmaSmem<TS_SQ, 1, row_stages<TS_SQ>()>::BYTES, StageTile<TS_SQ, 4>::BYTES));
            LACT_BIG_LDS(k_token_reduce_rows_dma<TS_SQ>, SM);
            LACT_LAUNCH_SMEM("k_token_reduce_rows_dma<128x128>", site, fl + frows, (k_token_reduce_rows_dma<TS_SQ>), gr, dim3(DMA_THREADS), SM, s, q);
          }
          rows->done = true;
        } else if (big) {
          constexpr int SM = cmax(DmaSmem<TS_NS, 1, row_stages<TS_NS>()>::BYTES, StageTile<TS_NS, 4>::BYTES);
          LACT_BIG_LDS(k_token_reduce_dma<TS_NS>, SM);
          LACT_LAUNCH_SMEM("k_token_reduce_dma<192x192>", site, fl, (k_token_reduce_dma<TS_NS>), g, dim3(DMA_THREADS), SM, s, pd);
        } else {
          constexpr int SM = cmax(DmaSmem<TS_SQ, 1, row_stages<TS_SQ>()>::BYTES, StageTile<TS_SQ, 4>::BYTES);
          LACT_BIG_LDS(k_token_reduce_dma<TS_SQ>, SM);
          LACT_LAUNCH_SMEM("k_token_reduce_dma<128x128>", site, fl, (k_token_reduce_dma<TS_SQ>), g, dim3(DMA_THREADS), SM, s, pd);
        }
        if (folded) return -1;
        if (main_tokens == tokens) return slots;
      }
    }
    // generic kernel: fp32, or fewer than 64 tokens
    const int rest = tokens - main_tokens;
    for (int i = 0; i < 3; ++i)
      for (int t = 0; t < p.job[i].nterms; ++t) {
        TokenReduceTerm& tt = p.job[i].t[t];
        tt.A = static_cast<const T*>(tt.A) + (size_t)main_tokens * tt.lda;
        tt.B = static_cast<const T*>(tt.B) + (size_t)main_tokens * tt.ldb;
      }
    const Split sp = main_tokens > 0 ? Split{1, ceil_div(rest, 32) * 32} : choose_split(rest, P.tiles * 3 * d.b, P.nsplit_max - 1);
    p.tokens = rest; p.split_len = sp.len;
    p.partial = partial + (size_t)slots * P.mat3;
    dim3 grid(P.tiles, sp.n, 3 * d.b);
    LACT_LAUNCH("k_token_reduce", site, 6.0 * rest * d.d * d.dh * d.b * jobs[0].nterms, (k_token_reduce<T, TSA>), grid, dim3(TSA::THREADS), s, p);
    if (direct) {   // add the tail to what the main part wrote
      LACT_LAUNCH("k_reduce_partials", "k_reduce_partials", 0.0, k_reduce_partials, flat, dim3(256), s, add_out, add_out, 1.f, partial, sp.n, (long long)P.mat3);
      return 0;
    }
    return slots + sp.n;
  }

  RenormParams renorm_params(int u, int ver_prev) const {
    RenormParams p;
    memset(&p, 0, sizeof(p));
    p.g = P.g;
    const bool replace = P.muon && d.muon_replaces_weight;
    p.base = d.prenorm ? main_(u) : wf(ver_prev);
    p.cw = replace ? 0.f : 1.f;
    p.u = P.muon ? usave(u) : dsave(u);
    p.raw = replace ? dsave(u) : nullptr;
    p.cr = replace ? 1.f : 0.f;
    p.n0 = n0();
    p.weight_norm = d.weight_norm;
    p.u_stacked = (P.muon && P.g.stacked) ? 1 : 0;
    p.eps_in_sqrt = d.renorm_eps_in_sqrt ? 1 : 0;
    return p;
  }

  // ------------------------------------------------------------------------------------------
  int forward(const float* w0, const float* w1, const float* w2, const T* q, const T* k, const T* v, const float* lr0,
              const float* lr1, const float* lr2, const float* mom, T* out, float* const w_out[3], float* const m_out[3],
              const float* const m_in[3]) {
    const dim3 rowgrid(ceil_div(P.g.maxrows(), 4), 3 * d.b);
    // what depends on the inputs only may start on the tail stream right here, beside the first kernels of the call
    hipEvent_t entry = nullptr;
    if (s_tail != s_main && side) {
      entry = side->event();
      (void)hipEventRecord(entry, s_main);
    }
    // carried momentum state: packed like every other state array (a device-to-device copy node when captured)
    if (P.state_in && P.nupd > 0)
      for (int j = 0; j < 3; ++j)
        if (hipMemcpyAsync(sv + P.s_min + (size_t)j * d.b * P.g.elems * 4, m_in[j], (size_t)d.b * P.g.elems * 4,
                           hipMemcpyDeviceToDevice, s) != hipSuccess)
          return fail("copy of the carried momentum state failed");
    {
      InitParams p;
      p.g = P.g; p.w[0] = w0; p.w[1] = w1; p.w[2] = w2; p.n0 = n0(); p.wf = wf(0);
      p.wc = P.bf16 ? (void*)wc(0) : nullptr;
      LACT_LAUNCH("k_init_state", "k_init_state", 0.0, (k_init_state<T>), rowgrid, dim3(256), s, p);
    }
    // mean of the momentum over the chunk of every update that weighs an earlier state (the first update of a
    // program has none unless the caller carried one in): they depend on the input only -- one launch up front
    if (P.momentum) {
      int u0 = P.state_in ? 0 : 1, ui = 0, n = 0;
      MomentumMeanRanges r;
      auto flush = [&]() {
        if (n > 0) LACT_LAUNCH("k_momentum_mean", "k_momentum_mean", 0.0, k_momentum_mean, dim3(d.b, n), dim3(256), s, mom, (long long)d.kv_len, r, mbar(u0));
        u0 += n; n = 0;
      };
      for (const auto& st : P.live) {
        if (st.kind != LACT_UPDATE) continue;
        if (ui++ < u0) continue;
        r.start[n] = st.start; r.len[n] = st.end - st.start;
        if (++n == 256) flush();
      }
      flush();
    }
    int ver = 0, u = 0;
    T* upd_z[3] = {nullptr, nullptr, nullptr};   // lr-scaled operands of the current update's gradient GEMMs
    long long upd_zbs = 0;
    bool side_used = false;
    // Apply steps only need their weight version, which is final once they are met in program order.  They are
    // held back and enqueued on the side stream at the point of the following update where the chip is least
    // busy -- in front of its Newton-Schulz kernels, which leave a quarter of the compute units idle -- or at
    // the end of the program.
    std::vector<std::pair<const lact_step_t*, int>> pending;   // (apply step, weight version)
    auto flush_applies = [&](bool beside_update) {
      if (pending.empty()) return;
      // with no update left to run beside, the caller's stream is the shortest way (no event hand-over)
      std::unique_ptr<OnSide> on_side;
      if (beside_update) {
        wait_for(s_side, s_main);
        side_used = true;
        on_side.reset(new OnSide(*this));
      }
      for (auto& pa : pending) {
        const lact_step_t& st = *pa.first;
        const int T_ = st.end - st.start, av = pa.second;
        HiddenParams hp = hidden_params(T_, q + (size_t)st.start * d.q_ld, d.q_ld, d.q_bs, nullptr, 0, 0, av);
        hp.O0 = h(0);
        launch_hidden(0, hp, av, T_);
        auto p = row_params<1>();
        set_term(p.t[0], h(0), d.dh, hbs(), wc(av, 1), d.dh, P.g.elems, d.dh);
        p.M = T_; p.N = d.d; p.out = out + (size_t)st.out_start * d.o_ld; p.ldo = d.o_ld; p.bso = d.o_bs;
        launch_row_gemm<T, true, 1, EPI_STORE>("apply_out", p, d.b, s, true);
      }
      pending.clear();
    };
    for (const auto& st : P.live) {
      const int T_ = st.end - st.start;
      if (st.kind == LACT_APPLY) {
        pending.emplace_back(&st, ver);
        if (s_side == s_main) flush_applies(false);   // one stream: plain program order
        continue;
      }
      // ---- update
      const T* kc = k + (size_t)st.start * d.k_ld;
      const T* vc = v + (size_t)st.start * d.v_ld;
      T* kl0 = scr<T>(P.t_kl[0]);
      T* kl2 = scr<T>(P.t_kl[1]);
      const long long klbs = (long long)P.Tcap * d.d;
      // k * lr0, k * lr2 depend on the inputs only and are first read by the token reduction: they are written on the
      // tail stream beside the hidden stage -- after everything enqueued so far (which includes the previous update's
      // reduction that read the same two buffers), the first update's already beside the state set-up of the call
      hipEvent_t kl_ready = nullptr;
      {
        const bool aside = s_tail != s_main && side;
        if (aside) {
          if (u == 0 && entry) (void)hipStreamWaitEvent(s_tail, entry, 0);
          else wait_for(s_tail, s_main);
          s = s_tail;
        }
        LACT_LAUNCH("k_lr_scale_rows", "update_lr_k", 0.0, (k_lr_scale_rows<T>), dim3((unsigned)(((long long)T_ * d.d / 4 + 255) / 256), d.b), dim3(256), s,
                    kc, d.k_ld, d.k_bs, lr0 + st.start, lr2 + st.start, (long long)d.kv_len, T_, d.d, kl0, kl2, klbs);
        if (aside) {
          kl_ready = side->event();
          (void)hipEventRecord(kl_ready, s_tail);
          s = s_main;
        }
      }
      {
        HiddenParams hp = hidden_params(T_, kc, d.k_ld, d.k_bs, vc, d.v_ld, d.v_bs, ver);
        hp.lr0 = lr0 + st.start; hp.lr1 = lr1 + st.start; hp.lr2 = lr2 + st.start; hp.bslr = d.kv_len;
        // operands of the three gradient GEMMs: dgate_before_act, hidden * lr1, dhidden_before_mul
        T* z0 = h(0); T* z1 = h(1); T* z2 = h(2);
        long long zbs = hbs();
        if (P.keep_pre) {
          // the unscaled operands stay in scratch (each region holds b * Tcap * dh elements: room for this stride)
          z0 = h(0); z1 = pre(u, 1); z2 = h(2); zbs = pre_bs(u);
          hp.O3 = pre(u, 3); hp.O4 = pre(u, 4); hp.O5 = pre(u, 5);
          hp.O6 = pre(u, 0); hp.O7 = pre(u, 2);
          hp.bso = zbs;
        }
        hp.O0 = z0; hp.O1 = z1; hp.O2 = z2;
        launch_hidden(1, hp, ver, T_);
        upd_z[0] = z0; upd_z[1] = z1; upd_z[2] = z2; upd_zbs = zbs;
      }
      // the pre-Muon gradient (= the momentum state) of the last update: read by nothing when Newton-Schulz output is
      // what enters the weights (the next update and its backward would read it; the caller gets its own copy)
      const bool d_unread = P.muon && !d.muon_replaces_weight && u + 1 == P.nupd;
      int dw_slots = 0;
      if (kl_ready) (void)hipStreamWaitEvent(s_main, kl_ready, 0);
      {
        TokenReduceJob jobs[3];
        memset(jobs, 0, sizeof(jobs));
        jobs[0].nterms = jobs[1].nterms = jobs[2].nterms = 1;
        jobs[0].M = d.dh; jobs[0].N = d.d;
        set_tr_term(jobs[0].t[0], upd_z[0], d.dh, upd_zbs, kl0, d.d, klbs);
        jobs[1].M = d.d; jobs[1].N = d.dh;
        set_tr_term(jobs[1].t[0], vc, d.v_ld, d.v_bs, upd_z[1], d.dh, upd_zbs);
        jobs[2].M = d.dh; jobs[2].N = d.d;
        set_tr_term(jobs[2].t[0], upd_z[2], d.dh, upd_zbs, kl2, d.d, klbs);
        // square shapes with Muon: the momentum step can ride in the reduction's epilogue (every tile exists for
        // every matrix, and the Newton-Schulz orientation is the packed one)
        PrepFold pf;
        pf.skip_d = false;
        const bool can_fold = kBf16 && kNsBf16 && P.muon && !P.g.stacked && d.d == d.dh;
        if (can_fold) {
          for (int j = 0; j < 3; ++j) pf.m_ext[j] = (u + 1 == P.nupd && P.momentum && m_out) ? m_out[j] : nullptr;
          pf.d_out = dsave(u); pf.m_prev = mprev(u); pf.skip_d = d_unread;
          pf.mbar = has_prev(u) ? mbar(u) : nullptr;
          pf.g16 = reinterpret_cast<uint16_t*>(g16(u)); pf.ss_part = scr<float>(P.t_ss);
          pf.clear.ptr = nullptr; pf.clear.n = 0;
          if (ns_all_fused()) pf.clear = ns_clear();
        }
        dw_slots = token_reduce("update_dw", jobs, T_, nullptr, nullptr, 0.f, can_fold ? &pf : nullptr);
      }
      const bool prep_folded = dw_slots < 0;
      const int ss_parts = prep_folded ? token_reduce_dma_tiles(d.d, d.dh) : P.nblk;
      if (!prep_folded) {
        MomentumPrepParams p;
        memset(&p, 0, sizeof(p));
        p.g = P.g; p.partial = scr<float>(P.t_partial); p.nsplit = dw_slots;
        p.m_prev = mprev(u);
        p.mbar = has_prev(u) ? mbar(u) : nullptr;
        p.d_out = d_unread ? nullptr : dsave(u);
        p.g16 = P.muon ? g16(u) : nullptr;
        p.ss_part = scr<float>(P.t_ss);
        p.round_partial_bf16 = P.bf16;
        if (u + 1 == P.nupd && P.momentum && m_out)
          for (int j = 0; j < 3; ++j) p.m_ext[j] = m_out[j];
        if (ns_all_fused()) p.clear = ns_clear();
        LACT_LAUNCH("k_momentum_prep", "k_momentum_prep", 0.0, (k_momentum_prep<TN>), dim3(P.nblk, 3 * d.b), dim3(256), s, p);
      }
      flush_applies(true);
      if (P.muon) {
        const bool scale_in_kernel = ns_all_fused();
        if (!scale_in_kernel) {
          NsScaleParams p;
          memset(&p, 0, sizeof(p));
          p.g = P.g; p.g16 = g16(u); p.ss_part = scr<float>(P.t_ss); p.nparts = ss_parts; p.norms = norms(u);
          p.xf = scr<float>(P.t_xf[0]); p.xb = xb(u, 0);
          p.u = P.S == 0 ? usave(u) : nullptr;
          p.plain_bf16 = d.ns_mode == LACT_NS_PLAIN_BF16;
          p.clear = ns_clear();
          LACT_LAUNCH("k_ns_scale", "k_ns_scale", 0.0, (k_ns_scale<TN>), dim3(P.nblk, P.g.ns_count()), dim3(256), s, p);
        }
        for (const NsBatch& B : P.nsb) {
          if (ns_fused_ok(B)) {
            if constexpr (kNsBf16) {
              NsFusedParams f;
              memset(&f, 0, sizeof(f));
              f.plain = d.ns_mode == LACT_NS_PLAIN_BF16;
              f.xf[0] = scr<float>(P.t_xf[0]) + B.xoff; f.xf[1] = scr<float>(P.t_xf[1]) + B.xoff;
              f.xb = xb(u, 0) + B.xoff; f.xb_it_stride = (long long)P.mat3;
              f.ab = ab(u, 0) + B.sqoff; f.bb = bb(u, 0) + B.sqoff; f.sq_it_stride = (long long)sq3();
              f.cab = scr<uint16_t>(P.t_ca) + B.sqoff;
              f.u_out = usave(u) + B.xoff;
              if (scale_in_kernel) {
                f.g16 = reinterpret_cast<const uint16_t*>(g16(u)) + B.xoff;
                f.ss_part = scr<float>(P.t_ss); f.nparts = ss_parts;
                f.part0 = B.first; f.part1 = (P.g.stacked && B.first == 0) ? 2 * d.b : -1;
                f.norms = norms(u) + B.first;
              }
              launch_ns_fused<false>(f, B);
            }
            continue;
          }
          for (int it = 0; it < P.S; ++it) {
            const bool last = it + 1 == P.S;
            NsIter I;
            I.n = B.n; I.r = B.r; I.c = B.c; I.nb_for_mask = B.nb; I.mask = B.mask; I.plain = d.ns_mode == LACT_NS_PLAIN_BF16;
            I.ca = P.coeffs[3 * it]; I.cb = P.coeffs[3 * it + 1]; I.cc = P.coeffs[3 * it + 2];
            I.xf_in = scr<float>(P.t_xf[it & 1]) + B.xoff; I.xb_in = xb(u, it) + B.xoff;
            I.ab = ab(u, it) + B.sqoff; I.bb = bb(u, it) + B.sqoff; I.cab = scr<TN>(P.t_ca) + B.sqoff;
            I.xf_out = last ? nullptr : scr<float>(P.t_xf[(it + 1) & 1]) + B.xoff;
            I.xb_out = last ? (void*)(scr<TN>(P.t_xbtmp) + B.xoff) : (void*)(xb(u, it + 1) + B.xoff);
            I.u_out = last ? usave(u) + B.xoff : nullptr;
            ns_iteration<TN>(I, s);
          }
        }
      }
      {
        RenormParams p = renorm_params(u, ver);
        p.main_out = d.prenorm ? main_(u + 1) : nullptr;
        // the fp32 copy of a weight version is the base of the next update (and of its backward): the last one has none
        // (with fp32 activations it is also what the apply steps read)
        p.wf_out = (P.bf16 && u + 1 == P.nupd) ? nullptr : wf(ver + 1);
        p.wc_out = P.bf16 ? (void*)wc(ver + 1) : nullptr;
        if (u + 1 == P.nupd && w_out)
          for (int j = 0; j < 3; ++j) p.w_ext[j] = w_out[j];
        if (P.muon && ns_fused_any()) p.poison = ns_error_word();
        LACT_LAUNCH("k_update_renorm", "k_update_renorm", 0.0, (k_update_renorm<T>), rowgrid, dim3(256), s, p);
      }
      ++ver;
      ++u;
    }
    flush_applies(false);
    if (side_used) wait_for(s_main, s_side);
    // final weights and momentum state: written by the last update's kernels; copied only when no update ran
    const dim3 eg((unsigned)((P.g.elems / 4 + 255) / 256), 3 * d.b);
    if (u == 0 && w_out && (w_out[0] || w_out[1] || w_out[2]))
      LACT_LAUNCH("k_unpack3", "k_unpack3", 0.0, k_unpack3, eg, dim3(256), s, wf(ver), P.g.elems, d.b, w_out[0], w_out[1], w_out[2]);
    if (m_out && (m_out[0] || m_out[1] || m_out[2])) {
      if (u > 0 && P.momentum) {
      } else
        for (int j = 0; j < 3; ++j)
          if (m_out[j]) LACT_LAUNCH("k_fill_f32", "k_fill_f32", 0.0, k_fill_f32, dim3((unsigned)((d.b * P.g.elems + 255) / 256)), dim3(256), s, m_out[j], 0.f, (long long)d.b * P.g.elems);
    }
    LACT_CHECK_LAUNCH();
    return 0;
  }

  // ------------------------------------------------------------------------------------------
  // Gradient rows of a token range are stored on first touch and accumulated on a repeat.  `force` (set when two
  // ranges of the program overlap without being equal) pre-zeroes the whole buffer and accumulates everywhere.
  struct Touched {
    std::vector<std::pair<int, int>> seen;
    bool force = false;
    bool accumulate(int a, int b) {
      bool hit = force;
      for (auto& iv : seen) hit = hit || (a < iv.second && iv.first < b);
      seen.emplace_back(a, b);
      return hit;
    }
  };
  // Rows of [0, len) that no step of `kind` touches, and whether any two of its ranges overlap partially.
  static std::vector<std::pair<int, int>> untouched(const std::vector<lact_step_t>& steps, int kind, int len, bool* partial) {
    std::vector<std::pair<int, int>> iv;
    for (auto& st : steps)
      if (st.kind == kind) iv.emplace_back(st.start, st.end);
    *partial = false;
    for (size_t i = 0; i < iv.size(); ++i)
      for (size_t j = i + 1; j < iv.size(); ++j)
        if (iv[i] != iv[j] && iv[i].first < iv[j].second && iv[j].first < iv[i].second) *partial = true;
    std::sort(iv.begin(), iv.end());
    std::vector<std::pair<int, int>> gaps;
    int pos = 0;
    for (auto& r : iv) {
      if (r.first > pos) gaps.emplace_back(pos, r.first);
      pos = std::max(pos, r.second);
    }
    if (pos < len) gaps.emplace_back(pos, len);
    if (*partial) gaps.assign(1, std::make_pair(0, len));
    return gaps;
  }
  struct ZeroList {
    ZeroSegments z;
    int n = 0;
    long long maxlen = 0;
    int nb;
    hipStream_t s;
    bool launched = false;
    ZeroList(int nb_, hipStream_t s_) : nb(nb_), s(s_) {}
    void flush() {
      if (n > 0 && maxlen > 0) {
        LACT_LAUNCH("k_zero_segments", "k_zero_segments", 0.0, k_zero_segments, dim3((unsigned)((maxlen + 4095) / 4096), nb, n), dim3(256), s, z);
        launched = true;
      }
      n = 0; maxlen = 0;
    }
    void add(void* ptr, long long bs, long long off, long long len) {
      if (!ptr || len <= 0) return;
      z.ptr[n] = static_cast<char*>(ptr); z.bs[n] = bs; z.off[n] = off; z.len[n] = len;
      maxlen = std::max(maxlen, len);
      if (++n == 16) flush();
    }
  };

  int backward(const T* q, const T* k, const T* v, const float* lr0, const float* lr1, const float* lr2, const float* mom,
               const T* dout, const float* const dwf[3], float* dw0, float* dw1, float* dw2, T* dq, T* dk, T* dv, float* dlr0,
               float* dlr1, float* dlr2, float* dmom) {
    (void)mom;
    const dim3 rowgrid(ceil_div(P.g.maxrows(), 4), 3 * d.b);
    const dim3 eg((unsigned)((P.g.elems / 4 + 255) / 256), 3 * d.b);
    const dim3 flat((unsigned)((P.mat3 / 4 + 255) / 256));
    float* gwcur = scr<float>(P.t_gwcur);
    float* gn0 = scr<float>(P.t_gn0);
    float* gmcarry = scr<float>(P.t_gmcarry);
    float* partial = scr<float>(P.t_partial);
    const long long gn0_n = (long long)3 * d.b * P.g.maxrows();
    // gn0 is written (not added to) by the first renorm backward; without any update the final kernel reads zeros
    bool gn0_written = false;
    if (P.nupd == 0) LACT_LAUNCH("k_fill_f32", "k_fill_f32", 0.0, k_fill_f32, dim3((unsigned)((gn0_n + 255) / 256)), dim3(256), s, gn0, 0.f, gn0_n);
    // gwcur: gradient w.r.t. the current weight version; "not valid" stands for zero (nothing written yet)
    bool gw_valid = dwf && (dwf[0] || dwf[1] || dwf[2]);
    if (gw_valid) LACT_LAUNCH("k_pack3", "k_pack3", 0.0, k_pack3, eg, dim3(256), s, gwcur, P.g.elems, d.b, dwf[0], dwf[1], dwf[2]);
    // every gradient output is written in full by this call: rows that no step touches are zeroed here.
    // Rows of dq, dk, dv and of the per-token arrays that no step writes are disjoint from everything the steps
    // write: nothing waits for them, and they are cleared on the side stream -- unless ranges overlap partially,
    // where the whole buffers start at zero and every step adds.  The momentum gradient is written by every
    // update but the first of the program (which has no earlier state to weigh).
    Touched seen_q, seen_kv, seen_m;
    const auto gaps_q = untouched(P.live, LACT_APPLY, d.q_len, &seen_q.force);
    const auto gaps_kv = untouched(P.live, LACT_UPDATE, d.kv_len, &seen_kv.force);
    std::vector<lact_step_t> later_updates;
    {
      bool first = true;
      for (auto& st : P.live)
        if (st.kind == LACT_UPDATE) {
          if (!first) later_updates.push_back(st);
          first = false;
        }
    }
    auto gaps_m = untouched(later_updates, LACT_UPDATE, d.kv_len, &seen_m.force);
    if (seen_kv.force) {
      seen_m.force = true;
      gaps_m.assign(1, std::make_pair(0, d.kv_len));
    }
    // momentum gradients: one launch at the end for all updates, unless token ranges of (later) updates repeat
    bool mg_each = seen_m.force;
    for (size_t i = 0; i < later_updates.size() && !mg_each; ++i)
      for (size_t j = i + 1; j < later_updates.size(); ++j)
        if (later_updates[i].start < later_updates[j].end && later_updates[j].start < later_updates[i].end) mg_each = true;
    // learning-rate gradients likewise; every update writes them
    bool lr_each = seen_kv.force;
    {
      std::vector<lact_step_t> ups;
      for (auto& st : P.live)
        if (st.kind == LACT_UPDATE) ups.push_back(st);
      for (size_t i = 0; i < ups.size() && !lr_each; ++i)
        for (size_t j = i + 1; j < ups.size(); ++j)
          if (ups[i].start < ups[j].end && ups[j].start < ups[i].end) lr_each = true;
    }
    std::vector<std::pair<int, int>> lr_ranges;   // met in descending order of the update index, all updates
    const size_t lrslot = (size_t)3 * P.lr_slots * d.b * P.Tcap;
    std::vector<int> mg_updates;
    int mg_parts = P.nblk;   // partial dots per matrix in a momentum-gradient slot (the same for every update)
    std::vector<std::pair<int, int>> mg_ranges;
    const bool rows_on_side = !seen_q.force && !seen_kv.force && s_side != s_main;
    auto zero_rows = [&](hipStream_t zs) {
      ZeroList zl(d.b, zs);
      const long long rowb = (long long)d.d * sizeof(T);
      for (auto& gp : gaps_q) zl.add(dq, (long long)d.q_len * rowb, gp.first * rowb, (gp.second - gp.first) * rowb);
      for (auto& gp : gaps_kv) {
        zl.add(dk, (long long)d.kv_len * rowb, gp.first * rowb, (gp.second - gp.first) * rowb);
        zl.add(dv, (long long)d.kv_len * rowb, gp.first * rowb, (gp.second - gp.first) * rowb);
        for (float* ptr : {dlr0, dlr1, dlr2})
          zl.add(ptr, (long long)d.kv_len * 4, gp.first * 4LL, (gp.second - gp.first) * 4LL);
      }
      for (auto& gp : gaps_m) zl.add(dmom, (long long)d.kv_len * 4, gp.first * 4LL, (gp.second - gp.first) * 4LL);
      zl.flush();
      return zl.launched;
    };
    if (!rows_on_side) zero_rows(s_main);
    // The apply steps run on the side stream.  Their weight gradients go to gw_side[version & 1] and are added
    // by the consumer of that version's gradient (the renorm backward of the update that made the version, or
    // the final kernel); `free_ev` orders the reuse of a gw_side buffer after its consumer.
    wait_for(s_side, s_main);
    float* gw_side[2] = {scr<float>(P.t_gwside[0]), scr<float>(P.t_gwside[1])};
    bool side_valid[2] = {false, false};
    hipEvent_t free_ev[2] = {nullptr, nullptr};
    hipEvent_t dw_done[2] = {nullptr, nullptr};   // newest weight-gradient kernel of the apply steps per buffer
    bool side_used = false;
    if (rows_on_side && zero_rows(s_side)) side_used = true;
    hipEvent_t main_dq_ev = nullptr;   // a dq GEMM on the side stream still reads the main chain's intermediates
    auto wait_main_dq = [&]() {
      if (main_dq_ev) (void)hipStreamWaitEvent(s_main, main_dq_ev, 0);
      main_dq_ev = nullptr;
    };
    // dk, dv and the learning-rate gradients of an update: nothing in the call waits for them, so they run on the
    // tail stream beside the rest of the chain.  They read the chain's token-major intermediates, the compute-type
    // gradient copy and the row partials: the chain waits for `tail_ev` before it writes any of those again.
    hipEvent_t tail_ev = nullptr;
    bool tail_used = false;
    auto wait_tail = [&]() {
      if (tail_ev) (void)hipStreamWaitEvent(s_main, tail_ev, 0);
      tail_ev = nullptr;
    };
    float* partial_side = scr<float>(P.t_partial_side);
    int ver = P.nupd, u = P.nupd;
    int carry_main = -1;       // index of the gwhat buffer holding the accumulator's gradient (pre-norm)
    bool gm_valid = false;     // gmcarry holds d loss / d (momentum state after update u-1)
    for (int si = (int)P.live.size() - 1; si >= 0; --si) {
      const lact_step_t& st = P.live[si];
      const int T_ = st.end - st.start;
      if (st.kind == LACT_APPLY) {
        const T* qc = q + (size_t)st.start * d.q_ld;
        const T* gc = dout + (size_t)st.out_start * d.do_ld;
        auto dw_jobs = [&](TokenReduceJob (&jobs)[3]) {
          memset(jobs, 0, sizeof(jobs));
          jobs[0].nterms = jobs[1].nterms = jobs[2].nterms = 1;
          jobs[0].M = d.dh; jobs[0].N = d.d;
          set_tr_term(jobs[0].t[0], h(1), d.dh, hbs(), qc, d.q_ld, d.q_bs);
          jobs[1].M = d.d; jobs[1].N = d.dh;
          set_tr_term(jobs[1].t[0], gc, d.do_ld, d.do_bs, h(0), d.dh, hbs());
          jobs[2].M = d.dh; jobs[2].N = d.d;
          set_tr_term(jobs[2].t[0], h(2), d.dh, hbs(), qc, d.q_ld, d.q_bs);
        };
        auto dq_gemm = [&]() {   // dq = gY0 W0 + gY2 W2
          auto p = row_params<2>();
          set_term(p.t[0], h(1), d.dh, hbs(), wc(ver, 0), d.d, P.g.elems, d.dh);
          set_term(p.t[1], h(2), d.dh, hbs(), wc(ver, 2), d.d, P.g.elems, d.dh);
          p.M = T_; p.N = d.d; p.out = dq + (size_t)st.start * d.d; p.ldo = d.d; p.bso = (long long)d.q_len * d.d;
          p.accumulate = seen_q.accumulate(st.start, st.end);
          launch_row_gemm<T, false, 2, EPI_STORE>("apply_bwd_dq", p, d.b, s, true);
        };
        if (ver == P.nupd) {
          // Applies of the newest weight version: the update chain cannot start before their weight gradients,
          // so they stay on the caller's stream (no event hand-over in the critical path); only dq, which nothing
          // waits for, goes to the side stream and reads this chain's intermediates.
          wait_main_dq();
          wait_tail();
          HiddenParams hp = hidden_params(T_, qc, d.q_ld, d.q_bs, gc, d.do_ld, d.do_bs, ver);
          hp.O0 = h(0); hp.O1 = h(1); hp.O2 = h(2);
          launch_hidden(2, hp, ver, T_);
          wait_for(s_side, s_main);
          TokenReduceJob jobs[3];
          dw_jobs(jobs);
          if (const int ns_ = token_reduce("apply_bwd_dw", jobs, T_, gwcur, gwcur, gw_valid ? 1.f : 0.f))
            LACT_LAUNCH("k_reduce_partials", "k_reduce_partials", 0.0, k_reduce_partials, flat, dim3(256), s, gwcur, gw_valid ? gwcur : nullptr, 1.f, partial, ns_, (long long)P.mat3);
          gw_valid = true;
          s = s_side;
          dq_gemm();
          s = s_main;
          if (side && s_side != s_main) {
            main_dq_ev = side->event();
            (void)hipEventRecord(main_dq_ev, s_side);
            side_used = true;
          }
          continue;
        }
        const int sb = ver & 1;
        if (!side_valid[sb] && free_ev[sb] && s_side != s_main) {
          (void)hipStreamWaitEvent(s_side, free_ev[sb], 0);
          free_ev[sb] = nullptr;
        }
        side_used = true;
        OnSide on_side(*this);
        HiddenParams hp = hidden_params(T_, qc, d.q_ld, d.q_bs, gc, d.do_ld, d.do_bs, ver);
        hp.O0 = h(0); hp.O1 = h(1); hp.O2 = h(2);
        launch_hidden(2, hp, ver, T_);
        TokenReduceJob jobs[3];
        dw_jobs(jobs);
        if (const int ns_ = token_reduce("apply_bwd_dw", jobs, T_, gw_side[sb], gw_side[sb], side_valid[sb] ? 1.f : 0.f))
          LACT_LAUNCH("k_reduce_partials", "k_reduce_partials", 0.0, k_reduce_partials, flat, dim3(256), s, gw_side[sb], side_valid[sb] ? gw_side[sb] : nullptr, 1.f, partial_side, ns_, (long long)P.mat3);
        side_valid[sb] = true;
        dw_done[sb] = side ? side->event() : nullptr;
        if (dw_done[sb] && s_side != s_main) (void)hipEventRecord(dw_done[sb], s_side);
        dq_gemm();
        continue;
      }
      // ---- update u-1: weights ver-1 -> ver
      --u;
      const int vprev = ver - 1;
      const int gw_idx = carry_main == 0 ? 1 : 0;
      float* gwhat = scr<float>(P.t_gwhat[gw_idx]);
      int cur = 0;  // which gxf/gxb buffer holds the running Newton-Schulz gradient
      {
        RenormParams p = renorm_params(u, vprev);
        p.gy = gw_valid ? gwcur : nullptr;
        const int sb = ver & 1;
        if (side_valid[sb]) {
          // wait for the apply steps' weight gradients only (their dq GEMMs may still be running)
          if (dw_done[sb] && s_side != s_main) (void)hipStreamWaitEvent(s_main, dw_done[sb], 0);
          p.gy2 = gw_side[sb];
        }
        p.carry_in = (d.prenorm && carry_main >= 0) ? scr<float>(P.t_gwhat[carry_main]) : nullptr;
        p.gw_hat = gwhat;
        p.gn0 = gn0; p.gn0_init = !gn0_written;
        gn0_written = true;
        p.clear = ns_clear();
        if (P.muon) { p.gxf = scr<float>(P.t_gxf[0]); p.gxb = scr<TN>(P.t_gxb[0]); }
        LACT_LAUNCH("k_renorm_bwd", "k_renorm_bwd", 0.0, (k_renorm_bwd<TN>), rowgrid, dim3(256), s, p);
        if (side_valid[sb]) {
          side_valid[sb] = false;
          if (side) {
            free_ev[sb] = side->event();
            (void)hipEventRecord(free_ev[sb], s_main);
          }
        }
      }
      if (d.prenorm) carry_main = gw_idx;
      // The backward of the Frobenius normalisation as the fused kernel's last stages: the partial dots always
      // (one batch, every matrix fused); the gradient in the compute type too when nothing else enters it (no
      // momentum state to carry, no raw-gradient term) and every matrix is held as it lies (square shapes).
      const bool dot_in_kernel = ns_all_fused() && P.nsb.size() == 1;
      const bool carry_here = P.momentum && (u > 0 || gm_valid);
      const bool prep_in_kernel = dot_in_kernel && kBf16 && !(P.muon && d.muon_replaces_weight) &&
                                  P.g.x_contiguous(0) && P.g.x_contiguous(1) && P.g.x_contiguous(2);
      const size_t mslot = (size_t)3 * d.b * std::max(P.nblk, 256);   // partial momentum dots of one update
      if (P.muon) {
        if (prep_in_kernel) wait_tail();   // the previous update's dk GEMM reads the gradient copy the fused kernel writes
        for (const NsBatch& B : P.nsb) {
          const int n = B.n, r = B.r, c = B.c;
          const long long xe = (long long)r * c, se = (long long)r * r;
          TN* sg = scr<TN>(P.t_sg) + B.sqoff;
          TN* gas = scr<TN>(P.t_gas) + B.sqoff;
          if (ns_fused_ok(B)) {
            if constexpr (kNsBf16) {
              NsFusedParams f;
              memset(&f, 0, sizeof(f));
              f.xb = xb(u, 0) + B.xoff; f.xb_it_stride = (long long)P.mat3;
              f.ab = ab(u, 0) + B.sqoff; f.bb = bb(u, 0) + B.sqoff; f.sq_it_stride = (long long)sq3();
              f.gxf[0] = scr<float>(P.t_gxf[0]) + B.xoff; f.gxf[1] = scr<float>(P.t_gxf[1]) + B.xoff;
              f.gxb[0] = scr<uint16_t>(P.t_gxb[0]) + B.xoff; f.gxb[1] = scr<uint16_t>(P.t_gxb[1]) + B.xoff;
              f.sg = reinterpret_cast<uint16_t*>(sg); f.gas = reinterpret_cast<uint16_t*>(gas);
              if (dot_in_kernel) {
                f.g16 = reinterpret_cast<const uint16_t*>(g16(u)) + B.xoff;
                f.dot_part = scr<float>(P.t_dot);
                f.norms = norms(u) + B.first;
                if (prep_in_kernel) {
                  f.gc = scr<uint16_t>(P.t_gc) + B.xoff;
                  if (carry_here) {   // as in k_grad_prep
                    f.gm_carry = gmcarry; f.carry_valid = gm_valid; f.carry_write = u > 0;
                    f.m_prev = u > 0 ? dsave(u - 1) : nullptr;
                    f.mbar = u > 0 ? mbar(u) : nullptr;
                    f.mdot_part = scr<float>(P.t_mdot) + (size_t)u * mslot;
                  }
                }
              }
              launch_ns_fused<true>(f, B);
            }
            continue;
          }
          int bc = 0;   // every batch starts from buffer 0 and ends in buffer S & 1
          for (int it = P.S - 1; it >= 0; --it) {
            const float ca = P.coeffs[3 * it], cb = P.coeffs[3 * it + 1], cc = P.coeffs[3 * it + 2];
            TN* gb = scr<TN>(P.t_gxb[bc]) + B.xoff;
            float* gf = scr<float>(P.t_gxf[bc]) + B.xoff;
            TN* xk = xb(u, it) + B.xoff;
            TN* ak = ab(u, it) + B.sqoff;
            TN* bk = bb(u, it) + B.sqoff;
            {  // Sg = G X^T + X G^T
              auto p = row_params<2>();
              set_term(p.t[0], gb, c, xe, xk, c, xe, c);
              set_term(p.t[1], xk, c, xe, gb, c, xe, c);
              p.M = r; p.N = r; p.out = sg; p.ldo = r; p.bso = se;
              launch_row_gemm<TN, true, 2, EPI_STORE>("ns_bwd_sg", p, n, s);
            }
            {  // gA + gA^T = b Sg + c (Sg A + A Sg)
              auto p = row_params<2>();
              set_term(p.t[0], sg, r, se, ak, r, se, r);
              set_term(p.t[1], ak, r, se, sg, r, se, r);
              p.M = r; p.N = r; p.out = gas; p.ldo = r; p.bso = se;
              p.aux = sg; p.ldaux = r; p.bsaux = se; p.alpha = cc; p.beta = cb;
              launch_row_gemm<TN, true, 2, EPI_AXPBY>("ns_bwd_ga", p, n, s);
            }
            {  // gX = a G + B G + (gA + gA^T) X
              auto p = row_params<2>();
              set_term(p.t[0], bk, r, se, gb, c, xe, r);
              set_term(p.t[1], gas, r, se, xk, c, xe, r);
              p.M = r; p.N = c; p.ldo = c; p.bso = xe;
              p.aux = gf; p.ldaux = c; p.bsaux = xe; p.alpha = 1.f; p.beta = ca;
              p.out = scr<float>(P.t_gxf[bc ^ 1]) + B.xoff;
              p.out_c = scr<TN>(P.t_gxb[bc ^ 1]) + B.xoff;
              launch_row_gemm<TN, false, 2, EPI_AXPBY_F32_DUAL>("ns_bwd_gx", p, n, s);
            }
            bc ^= 1;
          }
        }
        cur = P.S & 1;
        if (!dot_in_kernel && ns_dot_by_tiles()) {
          if constexpr (kNsBf16) {
            const NsBatch& B = P.nsb[0];
            NsTileDotParams q;
            q.gx = scr<float>(P.t_gxf[cur]) + B.xoff; q.g16 = reinterpret_cast<const uint16_t*>(g16(u)) + B.xoff;
            q.dot_part = scr<float>(P.t_dot); q.r = B.r; q.c = B.c;
            launch_ns_dot_tiles(q, B);
          }
        } else if (!dot_in_kernel) {
          NsDotParams dp;
          dp.g = P.g; dp.gx0 = scr<float>(P.t_gxf[cur]); dp.g16 = g16(u); dp.dot_part = scr<float>(P.t_dot);
          LACT_LAUNCH("k_ns_bwd_dot", "k_ns_bwd_dot", 0.0, (k_ns_bwd_dot<TN>), dim3(P.nblk, P.g.ns_count()), dim3(256), s, dp);
        }
      }
      if (!(P.muon && prep_in_kernel)) {
        wait_tail();   // the previous update's dk GEMM reads the gradient copy written here
        GradPrepParams p;
        memset(&p, 0, sizeof(p));
        p.g = P.g; p.muon = P.muon;
        p.gx0 = scr<float>(P.t_gxf[cur]); p.g16 = P.muon ? (const void*)g16(u) : nullptr; p.norms = norms(u);
        p.dot_part = scr<float>(P.t_dot); p.nparts = (P.muon && (dot_in_kernel || ns_dot_by_tiles())) ? ns_fused_nbm(P.nsb[0]) : P.nblk;
        p.gw_hat = gwhat; p.cr = (P.muon && d.muon_replaces_weight) ? 1.f : 0.f;
        p.gm_carry = (P.momentum && (u > 0 || gm_valid)) ? gmcarry : nullptr; p.carry_valid = gm_valid;
        p.carry_write = u > 0;
        p.m_prev = (P.momentum && u > 0) ? dsave(u - 1) : nullptr;
        p.mbar = (P.momentum && u > 0) ? mbar(u) : nullptr;
        p.gc = scr<T>(P.t_gc);
        p.mdot_part = scr<float>(P.t_mdot) + (size_t)u * mslot;
        if (P.muon && ns_fused_any()) p.poison = ns_error_word();
        LACT_LAUNCH("k_grad_prep", "k_grad_prep", 0.0, (k_grad_prep<T, TN>), dim3(P.nblk, 3 * d.b), dim3(256), s, p);
      }
      if (P.momentum) {
        gm_valid = true;
        // partial momentum dots per matrix: one per block of k_grad_prep, or one per tile of the fused kernel
        mg_parts = (P.muon && prep_in_kernel) ? ns_fused_nbm(P.nsb[0]) : P.nblk;
        // the gradient of the per-token momentum needs these dot products only: written by one launch at the end
        // (by one launch per update, in this order, when token ranges repeat and their shares add up)
        if (u > 0) {
          const bool acc = seen_m.accumulate(st.start, st.end);
          if (acc || mg_each) {
            MomentumMeanRanges r1;
            r1.start[0] = st.start; r1.len[0] = T_;
            LACT_LAUNCH("k_momentum_grad", "k_momentum_grad", 0.0, k_momentum_grad, dim3(d.b, 1), dim3(256), s, scr<float>(P.t_mdot) + (size_t)u * mslot,
                        0LL, mg_parts, d.b, dmom, (long long)d.kv_len, r1, acc ? 1 : 0);
          } else {
            mg_updates.push_back(u);
            mg_ranges.emplace_back(st.start, T_);
          }
        }
      }
      const T* kc = k + (size_t)st.start * d.k_ld;
      const T* vc = v + (size_t)st.start * d.v_ld;
      T* gcm = scr<T>(P.t_gc);
      T* g0 = gcm; T* g1 = gcm + (size_t)d.b * P.g.elems; T* g2 = gcm + (size_t)2 * d.b * P.g.elems;
      // lr-scaled operands of the forward's gradient GEMMs: kept by the forward, or written again by the hidden kernel
      T* z0 = h(3); T* z1 = h(4); T* z2 = h(5);
      long long zbs = hbs();
      {
        HiddenParams hp = hidden_params(T_, kc, d.k_ld, d.k_bs, vc, d.v_ld, d.v_bs, vprev);
        hp.lr0 = lr0 + st.start; hp.lr1 = lr1 + st.start; hp.lr2 = lr2 + st.start; hp.bslr = d.kv_len;
        hp.G0 = g0; hp.G1 = g1; hp.G2 = g2;
        hp.O0 = h(0); hp.O1 = h(1); hp.O2 = h(2); hp.O3 = h(3); hp.O4 = h(4); hp.O5 = h(5);
        hp.lrpart = scr<float>(P.t_lrpart) + (size_t)u * lrslot;
        hp.lrpart_stride = (long long)d.b * P.Tcap;
        hp.lrpart_mat_stride = (long long)P.lr_slots * d.b * P.Tcap;
        if (P.keep_pre) {
          hp.I0 = pre(u, 3); hp.I1 = pre(u, 4); hp.I2 = pre(u, 5); hp.bsi = pre_bs(u);
          hp.O3 = hp.O4 = hp.O5 = nullptr;
          z0 = pre(u, 0); z1 = pre(u, 1); z2 = pre(u, 2); zbs = pre_bs(u);
        }
        wait_main_dq();
        wait_tail();
        launch_hidden(P.keep_pre ? 4 : 3, hp, vprev, T_);
      }
      const bool acc_kv = seen_kv.accumulate(st.start, st.end);
      // worth a hand-over only when an earlier update's chain follows on the caller's stream
      // ... unless the token reduction of this update leaves most of the chip idle: then the GEMMs are worth more
      // inside its launch (below) than beside the chain (config 2, 48 reduction blocks: -1.4 %; config 4, 216: +1 %)
      bool lone_reduction = false;
      if constexpr (kBf16)
        lone_reduction = token_reduce_dma_tiles(d.d, d.dh) * 3 * d.b *
                             choose_split(T_, token_reduce_dma_tiles(d.d, d.dh) * 3 * d.b, P.nsplit_max - 1).n < 160;
      const bool use_tail = s_tail != s_main && u > 0 && !lone_reduction;
      if (use_tail) {
        wait_for(s_tail, s_main);
        s = s_tail;
      }
      // without that hand-over the two GEMMs share the launch of the token reduction below (when it runs on the
      // asynchronous-copy kernel; otherwise they are launched after it)
      RowCompanions rows_job;
      const bool rows_ride = !use_tail && kBf16;
      {  // dk = (dgate*lr0) G0 + (dh2*lr2) G2 + gG W0 + gH2 W2
        auto p = row_params<4>();
        set_term(p.t[0], z0, d.dh, zbs, g0, d.d, P.g.elems, d.dh);
        set_term(p.t[1], z2, d.dh, zbs, g2, d.d, P.g.elems, d.dh);
        set_term(p.t[2], h(0), d.dh, hbs(), wc(vprev, 0), d.d, P.g.elems, d.dh);
        set_term(p.t[3], h(2), d.dh, hbs(), wc(vprev, 2), d.d, P.g.elems, d.dh);
        p.M = T_; p.N = d.d; p.out = dk + (size_t)st.start * d.d; p.ldo = d.d; p.bso = (long long)d.kv_len * d.d;
        p.accumulate = acc_kv;
        if (use_tail || !kBf16) launch_row_gemm<T, false, 4, EPI_STORE>("update_bwd_dk", p, d.b, s, true);
        rows_job.r4 = p;
      }
      {  // dv = (hidden*lr1) G1^T + gDH W1^T
        auto p = row_params<2>();
        set_term(p.t[0], z1, d.dh, zbs, g1, d.dh, P.g.elems, d.dh);
        set_term(p.t[1], h(1), d.dh, hbs(), wc(vprev, 1), d.dh, P.g.elems, d.dh);
        p.M = T_; p.N = d.d; p.out = dv + (size_t)st.start * d.d; p.ldo = d.d; p.bso = (long long)d.kv_len * d.d;
        p.accumulate = acc_kv;
        if (use_tail || !kBf16) launch_row_gemm<T, true, 2, EPI_STORE>("update_bwd_dv", p, d.b, s, true);
        rows_job.r2 = p;
      }
      // learning-rate gradients: row partials of every update kept, one reduction launch at the end (one launch per
      // update, in this order, when token ranges repeat and their shares add up)
      if (lr_each) {
        MomentumMeanRanges r1;
        r1.start[0] = st.start; r1.len[0] = T_;
        LACT_LAUNCH("k_lr_reduce", "k_lr_reduce", 0.0, k_lr_reduce, dim3(ceil_div(T_, 256), d.b, 3), dim3(256), s,
                    scr<float>(P.t_lrpart) + (size_t)u * lrslot, 0LL, (long long)P.lr_slots * d.b * P.Tcap, (long long)d.b * P.Tcap, lr_parts(),
                    P.Tcap, dlr0, dlr1, dlr2, (long long)d.kv_len, r1, acc_kv ? 1 : 0);
      } else {
        lr_ranges.emplace_back(st.start, T_);
      }
      if (use_tail) {
        s = s_main;
        tail_ev = side->event();
        (void)hipEventRecord(tail_ev, s_tail);
        tail_used = true;
      }
      {
        TokenReduceJob jobs[3];
        memset(jobs, 0, sizeof(jobs));
        jobs[0].nterms = jobs[1].nterms = jobs[2].nterms = 1;
        jobs[0].M = d.dh; jobs[0].N = d.d;
        set_tr_term(jobs[0].t[0], h(0), d.dh, hbs(), kc, d.k_ld, d.k_bs);
        jobs[1].M = d.d; jobs[1].N = d.dh;
        set_tr_term(jobs[1].t[0], vc, d.v_ld, d.v_bs, h(1), d.dh, hbs());
        jobs[2].M = d.dh; jobs[2].N = d.d;
        set_tr_term(jobs[2].t[0], h(2), d.dh, hbs(), kc, d.k_ld, d.k_bs);
        const float pass = d.prenorm ? 0.f : ((P.muon && d.muon_replaces_weight) ? 0.f : 1.f);
        if (const int ns_ = token_reduce(rows_ride ? "update_bwd_dw_dk_dv" : "update_bwd_dw", jobs, T_, gwcur, gwhat, pass, nullptr,
                                         rows_ride ? &rows_job : nullptr))
          LACT_LAUNCH("k_reduce_partials", "k_reduce_partials", 0.0, k_reduce_partials, flat, dim3(256), s, gwcur, pass != 0.f ? gwhat : nullptr, pass, partial, ns_, (long long)P.mat3);
        gw_valid = true;
        if (rows_ride && !rows_job.done) {
          launch_row_gemm<T, false, 4, EPI_STORE>("update_bwd_dk", rows_job.r4, d.b, s, true);
          launch_row_gemm<T, true, 2, EPI_STORE>("update_bwd_dv", rows_job.r2, d.b, s, true);
        }
      }
      --ver;
    }
    if (!lr_ranges.empty()) {
      const int total = (int)lr_ranges.size();   // = updates; entry total - 1 - u belongs to update u
      for (int u0 = 0; u0 < total; u0 += 256) {
        const int n = std::min(256, total - u0);
        MomentumMeanRanges r;
        int longest = 0;
        for (int i = 0; i < n; ++i) {
          r.start[i] = lr_ranges[total - 1 - (u0 + i)].first; r.len[i] = lr_ranges[total - 1 - (u0 + i)].second;
          longest = std::max(longest, r.len[i]);
        }
        LACT_LAUNCH("k_lr_reduce", "k_lr_reduce", 0.0, k_lr_reduce, dim3(ceil_div(longest, 256), d.b, 3 * n), dim3(256), s,
                    scr<float>(P.t_lrpart) + (size_t)u0 * lrslot, (long long)lrslot, (long long)P.lr_slots * d.b * P.Tcap, (long long)d.b * P.Tcap,
                    lr_parts(), P.Tcap, dlr0, dlr1, dlr2, (long long)d.kv_len, r, 0);
      }
    }
    if (!mg_updates.empty()) {
      // deferred updates are all updates but the first, met in descending order: slot u - 1 of the launch is update u
      const size_t slot = (size_t)3 * d.b * std::max(P.nblk, 256);
      const int total = (int)mg_updates.size();
      for (int i0 = 0; i0 < total; i0 += 256) {
        const int n = std::min(256, total - i0);
        MomentumMeanRanges r;
        int umin = mg_updates[total - 1 - i0];
        for (int i = 0; i < n; ++i) {
          const int idx = total - 1 - (i0 + i);   // ascending update index
          r.start[i] = mg_ranges[idx].first; r.len[i] = mg_ranges[idx].second;
        }
        LACT_LAUNCH("k_momentum_grad", "k_momentum_grad", 0.0, k_momentum_grad, dim3(d.b, n), dim3(256), s, scr<float>(P.t_mdot) + (size_t)umin * slot,
                    (long long)slot, mg_parts, d.b, dmom, (long long)d.kv_len, r, 0);
      }
    }
    {
      FinishParams p;
      if (side_used) wait_for(s_main, s_side);
      if (tail_used) wait_tail();
      p.g = P.g; p.gw = gw_valid ? gwcur : nullptr;
      p.gw2 = side_valid[0] ? gw_side[0] : nullptr;
      p.carry = (d.prenorm && carry_main >= 0) ? scr<float>(P.t_gwhat[carry_main]) : nullptr;
      p.gn0 = gn0; p.n0 = n0(); p.w_init = wf(0);
      p.through_norms = d.detach_norms ? 0 : 1;
      p.out[0] = dw0; p.out[1] = dw1; p.out[2] = dw2;
      LACT_LAUNCH("k_finish_weight_grads", "k_finish_weight_grads", 0.0, k_finish_weight_grads, eg, dim3(256), s, p);
    }
    LACT_CHECK_LAUNCH();
    return 0;
  }
};

int check_ptrs(std::initializer_list<const void*> ps, const char* what) {
  for (const void* p : ps)
    if (!p) return fail(std::string("null pointer: ") + what);
  return 0;
}

}  // namespace

// ---- standalone Newton-Schulz ---------------------------------------------------------------
namespace {
struct NsPlan {
  MatGeom g;
  int r, c, nblk;
  size_t o_g16, o_ss, o_norm, o_xf[2], o_xb[2], o_ab, o_bb, o_ca, bytes;
  void build(int n, int rows, int cols) {
    // one "matrix kind" (index 0) of shape [rows, cols]: d = cols, dh = rows
    g.d = cols; g.dh = rows; g.nb = n; g.elems = (long long)rows * cols; g.stacked = 0;
    r = std::min(rows, cols); c = std::max(rows, cols);
    nblk = std::max(1, std::min(256, (int)((g.elems + 2047) / 2048)));
    Bump b;
    const size_t e = (size_t)n * g.elems;
    o_g16 = b.take(e * 4); o_ss = b.take((size_t)n * nblk * 4); o_norm = b.take((size_t)n * 4);
    o_xf[0] = b.take(e * 4); o_xf[1] = b.take(e * 4); o_xb[0] = b.take(e * 4); o_xb[1] = b.take(e * 4);
    o_ab = b.take((size_t)n * r * r * 4); o_bb = b.take((size_t)n * r * r * 4); o_ca = b.take((size_t)n * r * r * 4);
    bytes = b.off + 256;
  }
};
}  // namespace

namespace {
template <typename TN>
int newton_schulz_t(int32_t n, int32_t rows, int32_t cols, const float* gin, float* out, int32_t steps, const float* coeffs,
                    int32_t ns_mode, void* workspace, hipStream_t s) {
  const int plain_bf16 = ns_mode == LACT_NS_PLAIN_BF16;
  NsPlan P;
  P.build(n, rows, cols);
  char* ws = align256(workspace);
  // MatGeom treats index 0 as [dh, d] = [rows, cols]; launch with grid.y = n so z / nb == 0 throughout.
  MomentumPrepParams mp;
  memset(&mp, 0, sizeof(mp));
  mp.g = P.g; mp.partial = gin; mp.nsplit = 1; mp.d_out = reinterpret_cast<float*>(ws + P.o_xf[1]);
  mp.g16 = ws + P.o_g16; mp.ss_part = reinterpret_cast<float*>(ws + P.o_ss);
  // partial is indexed [s][3*nb][elems] with z < nb: the layout of gin ([n][elems]) matches for s = 0
  LACT_LAUNCH("k_momentum_prep", "k_momentum_prep", 0.0, (k_momentum_prep<TN>), dim3(P.nblk, n), dim3(256), s, mp);
  NsScaleParams sp;
  memset(&sp, 0, sizeof(sp));
  sp.g = P.g; sp.g16 = mp.g16; sp.ss_part = mp.ss_part; sp.nparts = P.nblk; sp.norms = reinterpret_cast<float*>(ws + P.o_norm);
  sp.xf = reinterpret_cast<float*>(ws + P.o_xf[0]); sp.xb = ws + P.o_xb[0];
  sp.u = steps == 0 ? out : nullptr; sp.plain_bf16 = plain_bf16;
  LACT_LAUNCH("k_ns_scale", "k_ns_scale", 0.0, (k_ns_scale<TN>), dim3(P.nblk, n), dim3(256), s, sp);
  for (int it = 0; it < steps; ++it) {
    const bool last = it + 1 == steps;
    NsIter I;
    I.n = n; I.r = P.r; I.c = P.c; I.nb_for_mask = n; I.mask = P.g.tall(0) ? 1 : 0; I.plain = plain_bf16;
    I.ca = coeffs[3 * it]; I.cb = coeffs[3 * it + 1]; I.cc = coeffs[3 * it + 2];
    I.xf_in = reinterpret_cast<float*>(ws + P.o_xf[it & 1]);
    I.xb_in = ws + P.o_xb[it & 1];
    I.ab = ws + P.o_ab; I.bb = ws + P.o_bb; I.cab = ws + P.o_ca;
    I.xf_out = last ? nullptr : reinterpret_cast<float*>(ws + P.o_xf[(it + 1) & 1]);
    I.xb_out = last ? nullptr : ws + P.o_xb[(it + 1) & 1];
    I.u_out = last ? out : nullptr;
    ns_iteration<TN>(I, s);
  }
  LACT_CHECK_LAUNCH();
  return 0;
}
}  // namespace


// ---- backward of the standalone Newton-Schulz: recomputes the iterates, then walks them backwards ------------
namespace {
struct NsBwdPlan {
  NsPlan f;
  size_t o_xb, o_ab, o_bb, o_gxf[2], o_gxb[2], o_sg, o_gas, o_dot, bytes;
  void build(int n, int rows, int cols, int steps) {
    f.build(n, rows, cols);
    Bump b;
    b.off = f.bytes;
    const size_t e = (size_t)n * f.g.elems, sq = (size_t)n * f.r * f.r, S = (size_t)std::max(1, steps);
    o_xb = b.take(S * e * 4); o_ab = b.take(S * sq * 4); o_bb = b.take(S * sq * 4);
    for (int i = 0; i < 2; ++i) { o_gxf[i] = b.take(e * 4); o_gxb[i] = b.take(e * 4); }
    o_sg = b.take(sq * 4); o_gas = b.take(sq * 4); o_dot = b.take((size_t)n * f.nblk * 4);
    bytes = b.off + 256;
  }
};

template <typename TN>
int newton_schulz_bwd_t(int32_t n, int32_t rows, int32_t cols, const float* gin, const float* dout, float* dg, int32_t steps,
                        const float* coeffs, int32_t ns_mode, void* workspace, hipStream_t s) {
  const int plain_bf16 = ns_mode == LACT_NS_PLAIN_BF16;
  NsBwdPlan P;
  P.build(n, rows, cols, steps);
  const NsPlan& F = P.f;
  char* ws = align256(workspace);
  const size_t e = (size_t)n * F.g.elems, sq = (size_t)n * F.r * F.r;
  auto xb = [&](int it) { return reinterpret_cast<TN*>(ws + P.o_xb) + (size_t)it * e; };
  auto ab = [&](int it) { return reinterpret_cast<TN*>(ws + P.o_ab) + (size_t)it * sq; };
  auto bb = [&](int it) { return reinterpret_cast<TN*>(ws + P.o_bb) + (size_t)it * sq; };
  // ---- forward again, keeping X_k, A_k, B_k
  MomentumPrepParams mp;
  memset(&mp, 0, sizeof(mp));
  mp.g = F.g; mp.partial = gin; mp.nsplit = 1; mp.d_out = nullptr;
  mp.g16 = ws + F.o_g16; mp.ss_part = reinterpret_cast<float*>(ws + F.o_ss);
  LACT_LAUNCH("k_momentum_prep", "k_momentum_prep", 0.0, (k_momentum_prep<TN>), dim3(F.nblk, n), dim3(256), s, mp);
  NsScaleParams sp;
  memset(&sp, 0, sizeof(sp));
  sp.g = F.g; sp.g16 = mp.g16; sp.ss_part = mp.ss_part; sp.nparts = F.nblk; sp.norms = reinterpret_cast<float*>(ws + F.o_norm);
  sp.xf = reinterpret_cast<float*>(ws + F.o_xf[0]); sp.xb = xb(0); sp.plain_bf16 = plain_bf16;
  LACT_LAUNCH("k_ns_scale", "k_ns_scale", 0.0, (k_ns_scale<TN>), dim3(F.nblk, n), dim3(256), s, sp);
  for (int it = 0; it + 1 < steps; ++it) {   // the last iterate itself is not needed
    NsIter I;
    I.n = n; I.r = F.r; I.c = F.c; I.nb_for_mask = n; I.mask = 0; I.plain = plain_bf16;
    I.ca = coeffs[3 * it]; I.cb = coeffs[3 * it + 1]; I.cc = coeffs[3 * it + 2];
    I.xf_in = reinterpret_cast<float*>(ws + F.o_xf[it & 1]); I.xb_in = xb(it);
    I.ab = ab(it); I.bb = bb(it); I.cab = ws + F.o_ca;
    I.xf_out = reinterpret_cast<float*>(ws + F.o_xf[(it + 1) & 1]); I.xb_out = xb(it + 1); I.u_out = nullptr;
    ns_iteration<TN>(I, s);
  }
  if (steps > 0) {   // A and B of the last iteration (its X' is the output the caller already has)
    const int it = steps - 1;
    const long long xe = (long long)F.r * F.c, se = (long long)F.r * F.r;
    auto p = row_params<1>();
    set_term(p.t[0], xb(it), F.c, xe, xb(it), F.c, xe, F.c);
    p.M = F.r; p.N = F.r; p.out = ab(it); p.ldo = F.r; p.bso = se;
    p.out2 = ws + F.o_ca; p.alpha2 = coeffs[3 * it + 2];
    launch_row_gemm<TN, true, 1, EPI_STORE>("ns_gram", p, n, s);
    auto q = row_params<1>();
    set_term(q.t[0], ws + F.o_ca, F.r, se, ab(it), F.r, se, F.r);
    q.M = F.r; q.N = F.r; q.out = bb(it); q.ldo = F.r; q.bso = se;
    q.aux = ab(it); q.ldaux = F.r; q.bsaux = se; q.alpha = 1.f; q.beta = coeffs[3 * it + 1];
    launch_row_gemm<TN, true, 1, EPI_AXPBY>("ns_poly", q, n, s);
  }
  // ---- the incoming gradient where Newton-Schulz holds its matrices
  float* gxf[2] = {reinterpret_cast<float*>(ws + P.o_gxf[0]), reinterpret_cast<float*>(ws + P.o_gxf[1])};
  TN* gxb[2] = {reinterpret_cast<TN*>(ws + P.o_gxb[0]), reinterpret_cast<TN*>(ws + P.o_gxb[1])};
  LACT_LAUNCH("k_to_ns_orientation", "k_to_ns_orientation", 0.0, (k_to_ns_orientation<TN>), dim3(F.nblk, n), dim3(256), s, F.g, dout, gxf[0], (void*)gxb[0]);
  TN* sg = reinterpret_cast<TN*>(ws + P.o_sg);
  TN* gas = reinterpret_cast<TN*>(ws + P.o_gas);
  const long long xe = (long long)F.r * F.c, se = (long long)F.r * F.r;
  int bc = 0;
  for (int it = steps - 1; it >= 0; --it) {
    const float ca = coeffs[3 * it], cb = coeffs[3 * it + 1], cc = coeffs[3 * it + 2];
    {  // Sg = G X^T + X G^T
      auto p = row_params<2>();
      set_term(p.t[0], gxb[bc], F.c, xe, xb(it), F.c, xe, F.c);
      set_term(p.t[1], xb(it), F.c, xe, gxb[bc], F.c, xe, F.c);
      p.M = F.r; p.N = F.r; p.out = sg; p.ldo = F.r; p.bso = se;
      launch_row_gemm<TN, true, 2, EPI_STORE>("ns_bwd_sg", p, n, s);
    }
    {  // gA + gA^T = b Sg + c (Sg A + A Sg)
      auto p = row_params<2>();
      set_term(p.t[0], sg, F.r, se, ab(it), F.r, se, F.r);
      set_term(p.t[1], ab(it), F.r, se, sg, F.r, se, F.r);
      p.M = F.r; p.N = F.r; p.out = gas; p.ldo = F.r; p.bso = se;
      p.aux = sg; p.ldaux = F.r; p.bsaux = se; p.alpha = cc; p.beta = cb;
      launch_row_gemm<TN, true, 2, EPI_AXPBY>("ns_bwd_ga", p, n, s);
    }
    {  // gX = a G + B G + (gA + gA^T) X
      auto p = row_params<2>();
      set_term(p.t[0], bb(it), F.r, se, gxb[bc], F.c, xe, F.r);
      set_term(p.t[1], gas, F.r, se, xb(it), F.c, xe, F.r);
      p.M = F.r; p.N = F.c; p.ldo = F.c; p.bso = xe;
      p.aux = gxf[bc]; p.ldaux = F.c; p.bsaux = xe; p.alpha = 1.f; p.beta = ca;
      p.out = gxf[bc ^ 1]; p.out_c = gxb[bc ^ 1];
      launch_row_gemm<TN, false, 2, EPI_AXPBY_F32_DUAL>("ns_bwd_gx", p, n, s);
    }
    bc ^= 1;
  }
  // ---- backward of X0 = G16 / (|G16| + 1e-7) and of the cast
  NsDotParams dp;
  dp.g = F.g; dp.gx0 = gxf[bc]; dp.g16 = ws + F.o_g16; dp.dot_part = reinterpret_cast<float*>(ws + P.o_dot);
  LACT_LAUNCH("k_ns_bwd_dot", "k_ns_bwd_dot", 0.0, (k_ns_bwd_dot<TN>), dim3(F.nblk, n), dim3(256), s, dp);
  GradPrepParams gp;
  memset(&gp, 0, sizeof(gp));
  gp.g = F.g; gp.muon = 1; gp.gx0 = gxf[bc]; gp.g16 = ws + F.o_g16; gp.norms = reinterpret_cast<float*>(ws + F.o_norm);
  gp.dot_part = dp.dot_part; gp.nparts = F.nblk; gp.gc = dg;
  LACT_LAUNCH("k_grad_prep", "k_grad_prep", 0.0, (k_grad_prep<float, TN>), dim3(F.nblk, n), dim3(256), s, gp);
  LACT_CHECK_LAUNCH();
  return 0;
}
}  // namespace

// ---- Newton-Schulz without a caller workspace: the workspace is a fixed array in device memory -------------
// Every GPU the library runs on holds its own copy of the array (at its own address) until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; the address it returns for the current
// device is what kernels and copies get.
static __device__ __align__(256) unsigned char scratch[LACT_NS_STATIC_WORKSPACE_BYTES];
namespace {
std::mutex g_static_ws_mutex;
void* g_static_ws[64] = {};   // per device: address of `scratch` there
// Address of the static workspace on the current device (looked up once per device), or null with the error set.
void* static_workspace() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= 64) {
    fail("static workspace: no current device (or device index beyond 63)");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_static_ws_mutex);
  if (!g_static_ws[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      fail(std::string("static workspace: hipGetSymbolAddress failed: ") + hipGetErrorString(e));
      return nullptr;
    }
    g_static_ws[dev] = ptr;
  }
  return g_static_ws[dev];
}
}  // namespace

extern "C" {

const char* lact_last_error(void) { return g_err.c_str(); }
int lact_version(void) { return 1; }

int lact_set_option(int32_t option, int32_t value) {
  std::lock_guard<std::mutex> lock(g_enqueue_mutex);
  if (option == LACT_OPT_NS_BARRIER_SPIN_LIMIT) {
    const long long was = g_ns_spin_limit;
    g_ns_spin_limit = value > 0 ? value : NS_FUSED_SPIN_LIMIT;
    return (int)std::min<long long>(was, 0x7fffffff);
  }
  if (option == LACT_OPT_KEEP_PREACTIVATIONS) {
    const int was = g_keep_pre;
    g_keep_pre = value < 0 ? -1 : (value != 0);
    return was;
  }
  if (option == LACT_OPT_PERSISTENT_TILES) {
    const int was = g_persist;
    g_persist = value;
    return was;
  }
  bool* flag = option == LACT_OPT_STREAM_OVERLAP ? &g_overlap : (option == LACT_OPT_FUSED_NEWTON_SCHULZ ? &g_fused_ns : nullptr);
  if (!flag) return fail("lact_set_option: unknown option");
  const int was = *flag ? 1 : 0;
  *flag = value != 0;
  return was;
}

// ---- layer pre- and post-processing -----------------------------------------------------------------
namespace {
int layer_geom(int32_t B, int32_t L, int32_t H, int32_t hd, LayerGeom* g) {
  if (B <= 0 || L <= 0 || H <= 0 || hd <= 0) return fail("layer: B, L, H, hd must be positive");
  if (hd % 4 || hd > 256 * LAYER_VEC_MAX) return fail("layer: head dim must be a multiple of 4 and at most 1024");
  g->B = B; g->L = L; g->H = H; g->hd = hd;
  return 0;
}
unsigned layer_row_blocks(const LayerGeom& g) { return (unsigned)(((long long)g.B * g.L * g.H + 3) / 4); }
unsigned layer_post_bwd_blocks(const LayerGeom& g) { return std::min(layer_row_blocks(g), 2048u); }
}  // namespace

int lact_layer_pre_forward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t l2norm, const void* qkv,
                           void* q, void* k, void* v, void* stream) {
  LayerPreParams p;
  memset(&p, 0, sizeof(p));
  if (layer_geom(B, L, H, hd, &p.g)) return -1;
  if (check_ptrs({qkv, q, k, v}, "layer pre tensors")) return -1;
  p.l2norm = l2norm; p.qkv = qkv; p.out[0] = q; p.out[1] = k; p.out[2] = v;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (act_dtype == LACT_BF16) LACT_LAUNCH("k_layer_pre", "layer_pre", 0.0, (k_layer_pre<uint16_t, false>), dim3(layer_row_blocks(p.g)), dim3(256), s, p);
  else if (act_dtype == LACT_F32) LACT_LAUNCH("k_layer_pre", "layer_pre", 0.0, (k_layer_pre<float, false>), dim3(layer_row_blocks(p.g)), dim3(256), s, p);
  else return fail("act_dtype must be LACT_BF16 or LACT_F32");
  LACT_CHECK_LAUNCH();
  return 0;
}

int lact_layer_pre_backward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t l2norm, const void* qkv,
                            const void* dq, const void* dk, const void* dv, void* dqkv, void* stream) {
  LayerPreParams p;
  memset(&p, 0, sizeof(p));
  if (layer_geom(B, L, H, hd, &p.g)) return -1;
  if (check_ptrs({qkv, dq, dk, dv, dqkv}, "layer pre backward tensors")) return -1;
  p.l2norm = l2norm; p.qkv = qkv; p.dout[0] = dq; p.dout[1] = dk; p.dout[2] = dv; p.dqkv = dqkv;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (act_dtype == LACT_BF16) LACT_LAUNCH("k_layer_pre_bwd", "layer_pre_bwd", 0.0, (k_layer_pre<uint16_t, true>), dim3(layer_row_blocks(p.g)), dim3(256), s, p);
  else if (act_dtype == LACT_F32) LACT_LAUNCH("k_layer_pre_bwd", "layer_pre_bwd", 0.0, (k_layer_pre<float, true>), dim3(layer_row_blocks(p.g)), dim3(256), s, p);
  else return fail("act_dtype must be LACT_BF16 or LACT_F32");
  LACT_CHECK_LAUNCH();
  return 0;
}

int lact_layer_lr_forward(int32_t B, int32_t L, int32_t H, int32_t rates_major, float base_lr_inv, const float* lr_raw, float* lr0, float* lr1,
                          float* lr2, const float* momentum_raw, float* momentum, void* stream) {
  LayerLrParams p;
  memset(&p, 0, sizeof(p));
  if (layer_geom(B, L, H, 4, &p.g)) return -1;
  if (check_ptrs({lr_raw, lr0, lr1, lr2}, "layer lr tensors")) return -1;
  if (momentum_raw && !momentum) return fail("momentum_raw given without momentum output");
  p.rates_major = rates_major != 0;
  p.base_lr_inv = base_lr_inv; p.lr_raw = lr_raw; p.lr[0] = lr0; p.lr[1] = lr1; p.lr[2] = lr2;
  p.mom_raw = momentum_raw; p.mom = momentum;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long long n = (long long)B * L * H;
  LACT_LAUNCH("k_layer_lr", "layer_lr", 0.0, (k_layer_lr<false>), dim3((unsigned)((n + 255) / 256)), dim3(256), s, p);
  LACT_CHECK_LAUNCH();
  return 0;
}

int lact_layer_lr_backward(int32_t B, int32_t L, int32_t H, int32_t rates_major, float base_lr_inv, const float* lr_raw, const float* dlr0,
                           const float* dlr1, const float* dlr2, float* dlr_raw, const float* momentum_raw,
                           const float* dmomentum, float* dmomentum_raw, void* stream) {
  LayerLrParams p;
  memset(&p, 0, sizeof(p));
  if (layer_geom(B, L, H, 4, &p.g)) return -1;
  if (check_ptrs({lr_raw, dlr_raw}, "layer lr backward tensors")) return -1;
  if (momentum_raw && !dmomentum_raw) return fail("momentum_raw given without dmomentum_raw output");
  p.rates_major = rates_major != 0;
  p.base_lr_inv = base_lr_inv; p.lr_raw = lr_raw; p.dlr[0] = dlr0; p.dlr[1] = dlr1; p.dlr[2] = dlr2; p.dlr_raw = dlr_raw;
  p.mom_raw = momentum_raw; p.dmom = dmomentum; p.dmom_raw = dmomentum_raw;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long long n = (long long)B * L * H;
  LACT_LAUNCH("k_layer_lr_bwd", "layer_lr_bwd", 0.0, (k_layer_lr<true>), dim3((unsigned)((n + 255) / 256)), dim3(256), s, p);
  LACT_CHECK_LAUNCH();
  return 0;
}

int lact_layer_post_forward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t use_norm, float eps,
                            const void* o, const float* norm_weight, const void* gate_raw, void* y, void* stream) {
  LayerPostParams p;
  memset(&p, 0, sizeof(p));
  if (layer_geom(B, L, H, hd, &p.g)) return -1;
  if (check_ptrs({o, y}, "layer post tensors")) return -1;
  p.eps = eps; p.use_norm = use_norm; p.o = o; p.w = norm_weight; p.gate_raw = gate_raw; p.y = y;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (act_dtype == LACT_BF16) LACT_LAUNCH("k_layer_post", "layer_post", 0.0, (k_layer_post<uint16_t, false>), dim3(layer_row_blocks(p.g)), dim3(256), s, p);
  else if (act_dtype == LACT_F32) LACT_LAUNCH("k_layer_post", "layer_post", 0.0, (k_layer_post<float, false>), dim3(layer_row_blocks(p.g)), dim3(256), s, p);
  else return fail("act_dtype must be LACT_BF16 or LACT_F32");
  LACT_CHECK_LAUNCH();
  return 0;
}

int32_t lact_layer_post_dw_rows(int32_t B, int32_t L, int32_t H) {
  LayerGeom g;
  if (layer_geom(B, L, H, 4, &g)) return -1;
  return (int32_t)layer_post_bwd_blocks(g) * 4;
}

int lact_layer_post_backward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t use_norm, float eps,
                             const void* o, const float* norm_weight, const void* gate_raw, const void* dy, void* d_o,
                             void* dgate_raw, float* dw_part, void* stream) {
  LayerPostParams p;
  memset(&p, 0, sizeof(p));
  if (layer_geom(B, L, H, hd, &p.g)) return -1;
  if (check_ptrs({o, dy, d_o}, "layer post backward tensors")) return -1;
  if (gate_raw && !dgate_raw) return fail("gate_raw given without dgate_raw output");
  p.eps = eps; p.use_norm = use_norm; p.o = o; p.w = norm_weight; p.gate_raw = gate_raw;
  p.dy = dy; p.d_o = d_o; p.dgate_raw = dgate_raw; p.dw_part = use_norm ? dw_part : nullptr;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (act_dtype == LACT_BF16) LACT_LAUNCH("k_layer_post_bwd", "layer_post_bwd", 0.0, (k_layer_post<uint16_t, true>), dim3(layer_post_bwd_blocks(p.g)), dim3(256), s, p);
  else if (act_dtype == LACT_F32) LACT_LAUNCH("k_layer_post_bwd", "layer_post_bwd", 0.0, (k_layer_post<float, true>), dim3(layer_post_bwd_blocks(p.g)), dim3(256), s, p);
  else return fail("act_dtype must be LACT_BF16 or LACT_F32");
  LACT_CHECK_LAUNCH();
  return 0;
}

int lact_check_async_error(void) {
  unsigned n = 0;
  hipError_t e = hipMemcpyFromSymbol(&n, HIP_SYMBOL(g_async_errors), sizeof(n), 0, hipMemcpyDeviceToHost);
  if (e != hipSuccess) return fail(std::string("lact_check_async_error: ") + hipGetErrorString(e));
  if (n == 0) return 0;
  const unsigned zero = 0;
  (void)hipMemcpyToSymbol(HIP_SYMBOL(g_async_errors), &zero, sizeof(zero), 0, hipMemcpyHostToDevice);
  // Whatever held the compute units may still be there: later calls use the unfused launches, which wait for nobody,
  // until the caller switches the fused kernel on again.
  {
    std::lock_guard<std::mutex> lock(g_enqueue_mutex);
    g_fused_ns = false;
  }
  g_err = std::to_string(n) + " barrier wait(s) of the fused Newton-Schulz kernel timed out on this device since the last check: "
          "the results of those steps are NaN (compute units held by another process or kernel).  "
          "LACT_OPT_FUSED_NEWTON_SCHULZ has been switched off: the calls that follow run three launches per iteration, "
          "same results; switch it on again (and, if the waits are merely slow, raise LACT_OPT_NS_BARRIER_SPIN_LIMIT) "
          "once the device is this process's alone";
  return (int)std::min<unsigned>(n, 0x7fffffffu);
}

// Back-to-back matrix instructions on every SIMD of every compute unit: the kernel of known matrix-pipe occupancy
// (all of it) that scales a matrix-busy counter of `rocprofv3 --pmc`, as a plain copy scales the byte counters.
__global__ __launch_bounds__(256) void k_mfma_calibration(int iters, float* out) {
  f32x16 acc[8];
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  bf16x8 a, b;
  for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(float)((threadIdx.x + j) & 7); b[j] = (__bf16)(float)((threadIdx.x * 3 + j) & 3); }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
  }
  float sum = 0.f;
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 16; ++j) sum += acc[i][j];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = sum;
}

int lact_mfma_calibration(int32_t blocks, int32_t iters, float* out, void* stream) {
  if (blocks <= 0 || iters <= 0 || !out) return fail("lact_mfma_calibration: bad arguments");
  hipLaunchKernelGGL(k_mfma_calibration, dim3(blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), iters, out);
  LACT_CHECK_LAUNCH();
  return 0;
}

int lact_profile_enable(int on) {
  g_prof.clear();
  g_prof.on = on != 0;
  return 0;
}

int lact_profile_report(char* buf, size_t cap) {
  if (!buf || cap == 0) return fail("null report buffer");
  hipError_t e = hipDeviceSynchronize();
  if (e != hipSuccess) return fail(std::string("synchronize failed: ") + hipGetErrorString(e));
  struct Agg { std::string kernel, site; long n = 0; double ms = 0, flops = 0; };
  std::vector<Agg> aggs;
  for (auto& r : g_prof.recs) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, r.e0, r.e1) != hipSuccess) continue;
    Agg* a = nullptr;
    for (auto& x : aggs)
      if (x.kernel == r.kernel && x.site == r.site) a = &x;
    if (!a) {
      aggs.push_back(Agg{r.kernel, r.site});
      a = &aggs.back();
    }
    a->n += 1;
    a->ms += ms;
    a->flops += r.flops;
  }
  std::string out = "[";
  for (size_t i = 0; i < aggs.size(); ++i) {
    char line[512];
    snprintf(line, sizeof(line), "%s{\"kernel\": \"%s\", \"site\": \"%s\", \"launches\": %ld, \"ms\": %.6f, \"flops\": %.6e}",
             i ? ", " : "", aggs[i].kernel.c_str(), aggs[i].site.c_str(), aggs[i].n, aggs[i].ms, aggs[i].flops);
    out += line;
  }
  out += "]";
  g_prof.clear();
  if (out.size() + 1 > cap) return fail("report buffer too small");
  memcpy(buf, out.c_str(), out.size() + 1);
  return 0;
}

int lact_query_sizes(const lact_desc_t* desc, size_t* saved_bytes, size_t* scratch_bytes) {
  Plan P;
  if (P.build(desc)) return -1;
  if (saved_bytes) *saved_bytes = P.saved_bytes;
  if (scratch_bytes) *scratch_bytes = P.scratch_bytes;
  return 0;
}

int lact_forward(const lact_desc_t* desc, const float* w0, const float* w1, const float* w2, const void* q, const void* k,
                 const void* v, const float* lr0, const float* lr1, const float* lr2, const float* momentum, void* out,
                 float* const w_out[3], float* const m_out[3], void* saved, void* scratch, void* stream) {
  return lact_forward_from_state(desc, w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum, nullptr, out, w_out, m_out, saved,
                                 scratch, stream);
}

int lact_forward_from_state(const lact_desc_t* desc, const float* w0, const float* w1, const float* w2, const void* q,
                            const void* k, const void* v, const float* lr0, const float* lr1, const float* lr2,
                            const float* momentum, const float* const m_in[3], void* out, float* const w_out[3],
                            float* const m_out[3], void* saved, void* scratch, void* stream) {
  Plan P;
  if (P.build(desc)) return -1;
  if (P.state_in && (!m_in || !m_in[0] || !m_in[1] || !m_in[2])) return fail("momentum_state_in set but a state pointer is null");
  if (!P.state_in && m_in) return fail("momentum state passed without momentum_state_in in the descriptor");
  if (check_ptrs({w0, w1, w2, q, out, saved, scratch}, "forward tensors")) return -1;
  if (P.nupd > 0 && check_ptrs({k, v, lr0, lr1, lr2}, "k, v, lr")) return -1;
  if (P.nupd > 0 && P.momentum && !momentum) return fail("use_momentum set but momentum is null");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  std::lock_guard<std::mutex> lock(g_enqueue_mutex);
#define LACT_FWD(T_, TN_)                                                                                           \
  {                                                                                                                 \
    Runner<T_, TN_> R(P, saved, scratch, s);                                                                        \
    return R.forward(w0, w1, w2, (const T_*)q, (const T_*)k, (const T_*)v, lr0, lr1, lr2, momentum, (T_*)out, w_out, \
                     m_out, m_in);                                                                                  \
  }
  const bool ns32 = P.d.ns_mode == LACT_NS_FP32;
  if (P.bf16 && !ns32) LACT_FWD(uint16_t, uint16_t)
  if (P.bf16 && ns32) LACT_FWD(uint16_t, float)
  if (!ns32) LACT_FWD(float, uint16_t)
  LACT_FWD(float, float)
#undef LACT_FWD
}

int lact_backward(const lact_desc_t* desc, const void* q, const void* k, const void* v, const float* lr0, const float* lr1,
                  const float* lr2, const float* momentum, const void* dout, const float* const dw_final[3], const void* saved,
                  void* scratch, float* dw0, float* dw1, float* dw2, void* dq, void* dk, void* dv, float* dlr0, float* dlr1,
                  float* dlr2, float* dmomentum, void* stream) {
  Plan P;
  if (P.build(desc)) return -1;
  if (P.d.forward_only) return fail("the forward ran with forward_only set: nothing was kept for a backward pass");
  if (check_ptrs({q, dout, saved, scratch, dw0, dw1, dw2, dq}, "backward tensors")) return -1;
  if (P.nupd > 0 && check_ptrs({k, v, lr0, lr1, lr2, dk, dv, dlr0, dlr1, dlr2}, "k, v, lr and their gradients")) return -1;
  if (P.nupd > 0 && P.momentum && (!momentum || !dmomentum)) return fail("use_momentum set but momentum or dmomentum is null");
  const int al = P.bf16 ? 8 : 4;
  if (P.d.do_ld % al || P.d.do_bs % al || P.d.do_ld < P.d.d) return fail("dout strides must keep 16-byte alignment");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  std::lock_guard<std::mutex> lock(g_enqueue_mutex);
#define LACT_BWD(T_, TN_)                                                                                            \
  {                                                                                                                  \
    Runner<T_, TN_> R(P, const_cast<void*>(saved), scratch, s);                                                      \
    return R.backward((const T_*)q, (const T_*)k, (const T_*)v, lr0, lr1, lr2, momentum, (const T_*)dout, dw_final,  \
                      dw0, dw1, dw2, (T_*)dq, (T_*)dk, (T_*)dv, dlr0, dlr1, dlr2, dmomentum);                        \
  }
  const bool ns32 = P.d.ns_mode == LACT_NS_FP32;
  if (P.bf16 && !ns32) LACT_BWD(uint16_t, uint16_t)
  if (P.bf16 && ns32) LACT_BWD(uint16_t, float)
  if (!ns32) LACT_BWD(float, uint16_t)
  LACT_BWD(float, float)
#undef LACT_BWD
}

size_t lact_newton_schulz_workspace_bytes(int32_t n, int32_t rows, int32_t cols, int32_t steps) {
  (void)steps;
  if (n <= 0 || rows <= 0 || cols <= 0) return 0;
  NsPlan P;
  P.build(n, rows, cols);
  return P.bytes;
}

int lact_newton_schulz(int32_t n, int32_t rows, int32_t cols, const float* gin, float* out, int32_t steps, const float* coeffs,
                       int32_t ns_mode, void* workspace, void* stream) {
  if (n <= 0 || rows <= 0 || cols <= 0 || n > 65535) return fail("bad Newton-Schulz shape");
  if (rows % 8 || cols % 8) return fail("rows and cols must be multiples of 8");
  if (steps < 0 || steps > 64 || (steps > 0 && !coeffs)) return fail("bad Newton-Schulz steps");
  if (ns_mode < 0 || ns_mode > 2) return fail("ns_mode must be 0, 1 or 2");
  if (!gin || !out || !workspace) return fail("null pointer: newton_schulz");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (ns_mode == LACT_NS_FP32) return newton_schulz_t<float>(n, rows, cols, gin, out, steps, coeffs, ns_mode, workspace, s);
  return newton_schulz_t<uint16_t>(n, rows, cols, gin, out, steps, coeffs, ns_mode, workspace, s);
}

size_t lact_newton_schulz_backward_workspace_bytes(int32_t n, int32_t rows, int32_t cols, int32_t steps) {
  if (n <= 0 || rows <= 0 || cols <= 0 || steps < 0) return 0;
  NsBwdPlan P;
  P.build(n, rows, cols, steps);
  return P.bytes;
}

int lact_newton_schulz_backward(int32_t n, int32_t rows, int32_t cols, const float* gin, const float* dout, float* dg,
                                int32_t steps, const float* coeffs, int32_t ns_mode, void* workspace, void* stream) {
  if (n <= 0 || rows <= 0 || cols <= 0 || n > 65535) return fail("bad Newton-Schulz shape");
  if (rows % 8 || cols % 8) return fail("rows and cols must be multiples of 8");
  if (steps < 0 || steps > 64 || (steps > 0 && !coeffs)) return fail("bad Newton-Schulz steps");
  if (ns_mode < 0 || ns_mode > 2) return fail("ns_mode must be 0, 1 or 2");
  if (!gin || !dout || !dg || !workspace) return fail("null pointer: newton_schulz_backward");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (ns_mode == LACT_NS_FP32) return newton_schulz_bwd_t<float>(n, rows, cols, gin, dout, dg, steps, coeffs, ns_mode, workspace, s);
  return newton_schulz_bwd_t<uint16_t>(n, rows, cols, gin, dout, dg, steps, coeffs, ns_mode, workspace, s);
}

size_t lact_newton_schulz_static_capacity(void) { return LACT_NS_STATIC_WORKSPACE_BYTES; }

int lact_newton_schulz_static(int32_t n, int32_t rows, int32_t cols, const float* gin, float* out, int32_t steps,
                              const float* coeffs, int32_t ns_mode, void* stream) {
  const size_t need = lact_newton_schulz_workspace_bytes(n, rows, cols, steps);
  if (need == 0) return fail("bad Newton-Schulz shape");
  if (need > LACT_NS_STATIC_WORKSPACE_BYTES)
    return fail("lact_newton_schulz_static: n x rows x cols needs " + std::to_string(need) + " workspace bytes, the static workspace holds " +
                std::to_string((size_t)LACT_NS_STATIC_WORKSPACE_BYTES) + " (use lact_newton_schulz with a caller workspace)");
  void* ws = static_workspace();
  if (!ws) return -1;
  return lact_newton_schulz(n, rows, cols, gin, out, steps, coeffs, ns_mode, ws, stream);
}

}  // extern "C"
