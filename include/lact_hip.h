/* C ABI of the MI355X large-chunk TTT library (liblact_hip.so).
 *
 * The reference has no FFI: its boundary for this path is a set of Python functions of tensors
 * called from the layers' forward().  Every entry point below is what a binding of that boundary
 * needs; none takes a torch type.  All pointers except `steps` and `ns_coeffs` are device
 * pointers; sizes are element counts unless a name says bytes; all calls enqueue work on `stream`
 * (a hipStream_t passed as void*) and return without synchronising.  Return value 0 = success,
 * negative = error; lact_last_error() gives the message of the calling thread's last failure.
 *
 * Layout (reference LLM layout, lact_llm/lact_model/ttt_operation.py:71-105):
 *   w0, w2: [b, dh, d]   w1: [b, d, dh]   fp32, contiguous
 *   q: [b, q_len, d]  k, v: [b, kv_len, d]   bf16 or fp32 (act_dtype), last dim contiguous,
 *      row stride *_ld and batch stride *_bs given in elements
 *   lr0, lr1, lr2, momentum: [b, kv_len] fp32 contiguous
 *   out: [b, out_len, d] act_dtype
 * d and dh must be multiples of 8; key and value dims are equal (every configuration of the
 * reference has dk == dv).
 */
#ifndef LACT_HIP_H
#define LACT_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { LACT_BF16 = 0, LACT_F32 = 1 };
enum { LACT_UPDATE = 0, LACT_APPLY = 1 };
/* Newton-Schulz numerics.  AUTOCAST: bf16 GEMM operands, fp32 accumulation and fp32 iterate, what
 * ttt_operation.py:30-66 computes under torch.autocast(bf16).  PLAIN_BF16: the iterate itself is
 * rounded to bf16 after every step, what the same code computes without autocast (:45 casts to bf16
 * and nothing casts back).  FP32: no bf16 anywhere (fp32 MFMA); not a reference mode, used to check
 * the closed-form backward against exact arithmetic. */
enum { LACT_NS_AUTOCAST = 0, LACT_NS_PLAIN_BF16 = 1, LACT_NS_FP32 = 2 };

/* One step of a test-time-training program.
 * UPDATE: one fast-weight update from k, v, lr, momentum rows [start, end)
 *         (ttt_operation.py:147-200; lact_nvs/lact_ttt.py:104-138).
 * APPLY:  out rows [out_start, out_start + end - start) = f_w(q rows [start, end))
 *         (ttt_operation.py:141-144; lact_nvs/lact_ttt.py:140-143).
 * The reference's schedules are all sequences of these: block-causal = apply,update per chunk then
 * a last apply (ttt_operation.py:124,202-212); bidirectional = update(all), apply(all)
 * (bidirectional_lact_layer.py:118-158); NVS = the TTTOperator list (lact_ttt.py:10,101);
 * AR video = apply, then update/apply pairs (ar_lact_swa_repeat.py:97-165). */
typedef struct lact_step {
  int32_t kind, start, end, out_start;
} lact_step_t;

typedef struct lact_desc {
  int32_t b, d, dh;
  int32_t q_len, kv_len, out_len;
  int32_t act_dtype;
  int32_t n_steps;
  const lact_step_t* steps;      /* host memory */
  int32_t ns_steps;              /* Newton-Schulz iterations; -1 = Muon off; 0 = cast + normalise only */
  const float* ns_coeffs;        /* host memory, 3*ns_steps floats (a,b,c per iteration;
                                    ttt_operation.py:51-57 or lact_ttt.py:51) */
  int32_t use_momentum;          /* ttt_operation.py:170-179 */
  int32_t prenorm;               /* ttt_operation.py:219-364 (un-normalised accumulator) */
  int32_t weight_norm;           /* ar_lact_swa_repeat.py:149-153 */
  int32_t detach_norms;          /* lact_ttt.py:96-98 */
  int32_t muon_replaces_weight;  /* bidirectional_lact_layer.py:139-146: w_hat = NS(dw) + dw */
  int32_t ns_mode;               /* LACT_NS_* */
  int64_t q_bs, k_bs, v_bs, o_bs, do_bs;
  int32_t q_ld, k_ld, v_ld, o_ld, do_ld;
  /* The two places where the fused-kernel driver differs in semantics (ttt_operation_fused_kernel.py): */
  int32_t muon_stacked;          /* Newton-Schulz on cat(dw0, dw2) [2dh, d] and on dw1 (:168-170, :308-310) */
  int32_t renorm_eps_in_sqrt;    /* y = w / sqrt(|w|^2 + eps) * n0 (:172-173; l2norm_triton_kernels.py:205-214) */
  /* No lact_backward call follows (inference, torch.no_grad): the forward keeps no activations for it, `saved` is
   * smaller, and lact_backward refuses the descriptor.  No counterpart in the reference, where autograd decides. */
  int32_t forward_only;
  /* The first update starts from a momentum state carried in by the caller (lact_forward_from_state) instead of
   * zero: ar_lact_swa_repeat_sp.py:215-217,266-269,309-317.  Needs use_momentum and forward_only. */
  int32_t momentum_state_in;
} lact_desc_t;

const char* lact_last_error(void);
int lact_version(void);

/* Bytes of the two caller-owned buffers: `saved` lives from forward to backward (fast-weight
 * versions, momentum states, Newton-Schulz iterates); `scratch` only during one call. */
int lact_query_sizes(const lact_desc_t* desc, size_t* saved_bytes, size_t* scratch_bytes);

/* Whole forward of one program.  Replaces block_causal_lact_swiglu / prenorm_block_causal_lact_swiglu
 * (ttt_operation.py:71-214, 219-364), their fused-kernel twins (ttt_operation_fused_kernel.py:67-338),
 * bidirectional_lact_swiglu (bidirectional_lact_layer.py:74-160),
 * fast_weight_swish_glu_weight_norm_mini_batch_apply (lact_ttt.py:71-147) and the
 * ar_fast_weight_swish_glu_weight_norm_mini_batch family (ar_lact_swa_repeat.py:23-296).
 * w_out[3] / m_out[3] (each nullable, fp32, shapes of w0,w1,w2) receive the final fast weights and
 * momentum states (lact_ttt.py:147; ar_lact_swa_repeat_sp.py:339). */
int lact_forward(const lact_desc_t* desc, const float* w0, const float* w1, const float* w2, const void* q,
                 const void* k, const void* v, const float* lr0, const float* lr1, const float* lr2,
                 const float* momentum, void* out, float* const w_out[3], float* const m_out[3], void* saved,
                 void* scratch, void* stream);

/* lact_forward with the momentum states of an earlier call carried in: m_in[3] (fp32, shapes of w0,w1,w2) is what
 * that call returned through m_out.  Replaces ar_fast_weight_swish_glu_weight_norm_mini_batch_inference_with_momentum
 * (ar_lact_swa_repeat_sp.py:197-339), whose caller keeps the states between denoising steps (:998-1053).
 * desc->momentum_state_in must be set (and m_in null when it is not); inference only. */
int lact_forward_from_state(const lact_desc_t* desc, const float* w0, const float* w1, const float* w2, const void* q,
                            const void* k, const void* v, const float* lr0, const float* lr1, const float* lr2,
                            const float* momentum, const float* const m_in[3], void* out, float* const w_out[3],
                            float* const m_out[3], void* saved, void* scratch, void* stream);

/* Backward of the same program (the reference relies on autograd; closed forms as in
 * lact_triton_kernels/lact_swiglu_ffn.py:46-76, lact_fw_grad.py:61-156, l2norm_triton_kernels.py:106-172).
 * dout: gradient of `out` (act_dtype, strides do_ld/do_bs); dw_final[3]: gradient of the returned
 * final weights (nullable).  Outputs: dw0,dw1,dw2 fp32; dq,dk,dv act_dtype contiguous [b,len,d];
 * dlr0..2, dmomentum fp32 [b,kv_len].  Every element of every output is written: rows no step touches
 * are set to zero, rows used by several steps hold the sum; the caller need not clear anything. */
int lact_backward(const lact_desc_t* desc, const void* q, const void* k, const void* v, const float* lr0,
                  const float* lr1, const float* lr2, const float* momentum, const void* dout,
                  const float* const dw_final[3], const void* saved, void* scratch, float* dw0, float* dw1,
                  float* dw2, void* dq, void* dk, void* dv, float* dlr0, float* dlr1, float* dlr2,
                  float* dmomentum, void* stream);

/* zeropower_via_newtonschulz5 (ttt_operation.py:30-66; with a repeated coefficient triple:
 * lact_ttt.py:33-67, functions.py:38-72).  g, out: [n, rows, cols] fp32. */
size_t lact_newton_schulz_workspace_bytes(int32_t n, int32_t rows, int32_t cols, int32_t steps);
int lact_newton_schulz(int32_t n, int32_t rows, int32_t cols, const float* g, float* out, int32_t steps,
                       const float* coeffs, int32_t ns_mode, void* workspace, void* stream);

/* Backward of lact_newton_schulz (in the reference autograd differentiates ttt_operation.py:30-66 / lact_ttt.py:33-67):
 * dg = d loss / d g from dout = d loss / d out; g, dout, dg: [n, rows, cols] fp32.  Recomputes the iterates from g (same
 * steps, coeffs, ns_mode as the forward call), then walks them backwards in closed form. */
size_t lact_newton_schulz_backward_workspace_bytes(int32_t n, int32_t rows, int32_t cols, int32_t steps);
int lact_newton_schulz_backward(int32_t n, int32_t rows, int32_t cols, const float* g, const float* dout, float* dg,
                                int32_t steps, const float* coeffs, int32_t ns_mode, void* workspace, void* stream);

/* lact_newton_schulz for callers that cannot allocate device memory or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The workspace is
 * a fixed array of LACT_NS_STATIC_WORKSPACE_BYTES in device memory that the library holds on every GPU it runs on
 * until the process ends; the call allocates nothing.  Shapes whose lact_newton_schulz_workspace_bytes exceed it are
 * refused (return value < 0, message in lact_last_error).  Every call on a GPU uses that GPU's one array: calls that
 * overlap on one GPU (two streams, two threads) race; calls on one stream are ordered by the stream.  Same kernels
 * and same results, bit for bit, as lact_newton_schulz.  The first call on a device looks up the array's address and
 * sets kernel attributes: make one call outside any graph capture before capturing one. */
#define LACT_NS_STATIC_WORKSPACE_BYTES (32u << 20)
size_t lact_newton_schulz_static_capacity(void);
int lact_newton_schulz_static(int32_t n, int32_t rows, int32_t cols, const float* g, float* out, int32_t steps,
                              const float* coeffs, int32_t ns_mode, void* stream);

/* ---- Layer pre- and post-processing (the tensor code of the layer classes around the operation, one pass each;
 * in the reference a chain of PyTorch ops in the layers' forward, with autograd for the backward).
 * act_dtype as above; head dim a multiple of 4, at most 1024.  All buffers contiguous.
 *
 * pre: qkv [B, L, 3, H, hd] (output of the layer's to_qkv projection) -> q, k, v [(B H), L, hd]:
 *      silu, L2 norm of q and k per head (x / (|x| + 1e-5)) when l2norm, head layout
 *      (bidirectional_lact_layer.py:231-244; causal_lact_with_sliding_window_attn.py:313-322). */
int lact_layer_pre_forward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t l2norm,
                           const void* qkv, void* q, void* k, void* v, void* stream);
int lact_layer_pre_backward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t l2norm,
                            const void* qkv, const void* dq, const void* dk, const void* dv, void* dqkv,
                            void* stream);
/* lr: lr_raw fp32 (output of lr_proj) -> lr0, lr1, lr2 [(B H), L] = softplus(raw + base_lr_inv); lr_raw is
 *     [B, L, H, 3] ('b l (h lrs d)') when rates_major == 0 and [B, L, 3, H] ('b l (lrs h d)', lact_ttt.py:213-216) else;
 *     momentum_raw [B, L, H] fp32 (nullable; output of the linear map of momentum_proj) -> sigmoid, [(B H), L]
 *     (bidirectional_lact_layer.py:248-256; causal_lact_with_sliding_window_attn.py:326-345). */
int lact_layer_lr_forward(int32_t B, int32_t L, int32_t H, int32_t rates_major, float base_lr_inv, const float* lr_raw, float* lr0,
                          float* lr1, float* lr2, const float* momentum_raw, float* momentum, void* stream);
int lact_layer_lr_backward(int32_t B, int32_t L, int32_t H, int32_t rates_major, float base_lr_inv, const float* lr_raw,
                           const float* dlr0, const float* dlr1, const float* dlr2, float* dlr_raw,
                           const float* momentum_raw, const float* dmomentum, float* dmomentum_raw, void* stream);
/* post: o [(B H), L, hd] (output of the operation) -> y [B, L, H*hd]: RMSNorm over the head dim with weight
 *      norm_weight [hd] fp32 (nullable = ones) when use_norm, times silu(gate_raw [B, L, H]) when gate_raw is
 *      given, head layout (bidirectional_lact_layer.py:268-270; causal_lact_with_sliding_window_attn.py:351-357).
 *      The backward writes lact_layer_post_dw_rows(B, L, H) partial rows of the weight gradient into
 *      dw_part [rows][hd] fp32 (the caller sums them), d_o and dgate_raw. */
int lact_layer_post_forward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t use_norm,
                            float eps, const void* o, const float* norm_weight, const void* gate_raw, void* y,
                            void* stream);
int32_t lact_layer_post_dw_rows(int32_t B, int32_t L, int32_t H);
int lact_layer_post_backward(int32_t act_dtype, int32_t B, int32_t L, int32_t H, int32_t hd, int32_t use_norm,
                             float eps, const void* o, const float* norm_weight, const void* gate_raw,
                             const void* dy, void* d_o, void* dgate_raw, float* dw_part, void* stream);

/* Execution options (process-wide; no counterpart in the reference, where PyTorch enqueues the whole layer on one
 * stream as separate kernels).  The switches are on by default and change no result bit.
 *   LACT_OPT_STREAM_OVERLAP: the apply steps of a program do not depend on the update chain that runs beside
 *     them, and nothing in a call waits for dk, dv or the learning-rate gradients of an update; lact_forward /
 *     lact_backward enqueue them on two library-owned streams (default priority, per device, created on first
 *     use) that are forked from and joined back into the caller's stream with events, so the call as a whole
 *     stays asynchronous and ordered on the caller's stream.
 *   LACT_OPT_FUSED_NEWTON_SCHULZ: all Newton-Schulz iterations of an update (and of its backward) run as one
 *     kernel whose blocks meet at per-matrix barriers (bf16; rows and columns multiples of 192, of 128, or rows of
 *     128 and columns of 64; at most 8 iterations); otherwise three GEMM launches per iteration.
 *   LACT_OPT_NS_BARRIER_SPIN_LIMIT: how many polls a block of the fused Newton-Schulz kernel waits at a barrier
 *     before it gives up (value <= 0 restores the default, a fraction of a second).  A block that gives up raises
 *     an error word and goes on, so every kernel always ends; the step's results (weights, outputs that depend on
 *     them, gradients) are then NaN.  Meant for tests of that path.
 *   LACT_OPT_PERSISTENT_TILES: the hidden-stage kernels (bf16, d a multiple of 64) run as one block per compute unit
 *     that walks its share of the tiles, the copy waves running ahead into the next tile while the matrix waves run
 *     the previous tile's epilogue; otherwise one tile per block.  Same arithmetic, same bits.  The value is a mask:
 *     bit 0 the apply's hidden stage, bit 1 the update's, bit 2 the apply backward's.  Default: 1.  The update's
 *     hidden stage, whose epilogue writes up to eight arrays, measured slower this way; the apply backward's measured
 *     2 % faster as a kernel but runs beside other kernels on a second stream, where a launch that holds every
 *     compute unit until its last tile costs the step more than it saves.
 *   LACT_OPT_KEEP_PREACTIVATIONS: 1: the update's forward keeps its rounded pre-activations and lr-scaled operands
 *     for the backward (bf16, d and dh multiples of 64), 0: the backward recomputes them, -1 (default): by shape
 *     (kept when d > 128).  Same bits either way, except the learning-rate gradients (fp32 sums over tiles of another
 *     width: 1e-7).  Read when a call is planned: set it before the
 *     forward and leave it until that forward's backward has been enqueued (the two must agree on what was saved).
 * Returns the previous value (0 / 1, or the previous limit), or -1 for an unknown option. */
enum { LACT_OPT_STREAM_OVERLAP = 0, LACT_OPT_FUSED_NEWTON_SCHULZ = 1, LACT_OPT_NS_BARRIER_SPIN_LIMIT = 2, LACT_OPT_PERSISTENT_TILES = 3, LACT_OPT_KEEP_PREACTIVATIONS = 4 };
int lact_set_option(int32_t option, int32_t value);

/* Errors that only the device notices.  A block of the fused Newton-Schulz kernel that gives up at a barrier (see
 * LACT_OPT_NS_BARRIER_SPIN_LIMIT) turns the step's results into NaN and adds one to a per-device counter that no
 * call clears.  lact_check_async_error copies that counter of the current device to the host (a synchronous copy: call
 * it once the stream the steps ran on has been synchronised), resets it and returns it: 0 = nothing happened, > 0 =
 * that many waits timed out since the last check (message in lact_last_error; LACT_OPT_FUSED_NEWTON_SCHULZ is then
 * switched off, so that the calls that follow cannot time out again, until the caller switches it back on), < 0 =
 * the check itself failed.  No
 * counterpart in the reference, whose kernels never wait for each other.  The fused kernel is only used on a device
 * with at least 256 compute units (its groups must be resident as a whole); elsewhere the unfused launches run. */
int lact_check_async_error(void);

/* Per-launch timing with HIP events on the caller's stream (no counterpart in the reference, which
 * times with wall-clock prints, lact_ar_video/minVid/train.py:458-460).  While enabled every kernel
 * launch of lact_forward / lact_backward is bracketed by two events; lact_profile_report synchronises
 * the device, writes a JSON array of {kernel, site, launches, ms, flops} into buf and resets the
 * records.  Not thread-safe; meant for benchmarking. */
int lact_profile_enable(int on);
/* Calibration kernel for matrix-pipe counters (`rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES ...`): `blocks` workgroups of
 * four waves that issue nothing but bf16 matrix instructions, `iters` x 8 each; out: blocks * 256 floats.  What the
 * counter reads for it is the reading of a fully busy matrix pipe.  No counterpart in the reference. */
int lact_mfma_calibration(int32_t blocks, int32_t iters, float* out, void* stream);
int lact_profile_report(char* buf, size_t cap);

#ifdef __cplusplus
}
#endif
#endif
