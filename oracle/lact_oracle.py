"""CPU oracle for the large-chunk SwiGLU fast-weight TTT operation (LaCT).

TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP path is compared with; it is
imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg and by
nothing else.  The product (lact_amd/) never imports it and has no CPU fallback.

It is a from-scratch restatement, in plain PyTorch with every dtype cast written out, of
the reference's non-fused operation:

  * lact_llm/lact_model/ttt_operation.py:5-17      silu_backprop
  * lact_llm/lact_model/ttt_operation.py:20-27     l2_norm
  * lact_llm/lact_model/ttt_operation.py:30-66     zeropower_via_newtonschulz5 (5-coefficient table)
  * lact_llm/lact_model/ttt_operation.py:71-214    block_causal_lact_swiglu (post-norm)
  * lact_llm/lact_model/ttt_operation.py:219-364   prenorm_block_causal_lact_swiglu
  * minimal_implementations/causal_lact_with_sliding_window_attn.py:84-211  (same op, other arg order)
  * minimal_implementations/bidirectional_lact_layer.py:74-160  bidirectional_lact_swiglu
  * lact_nvs/lact_ttt.py:33-67,71-147              classic NS + update/apply program, transposed layout
  * lact_ar_video/minVid/models/blocks/ar_lact_swa_repeat.py:23-168,172-296 and
    ar_lact_swa_repeat_sp.py:28-193                AR-video update-then-apply schedules

All variants are one interpreter (`run_program`) over a list of UPDATE / APPLY steps; the
named entry points only build that list and the flags.

Numerics.  `Numerics(autocast=True)` reproduces what the reference computes on a GPU under
`torch.autocast("cuda", dtype=bfloat16)` in eager mode: every matmul rounds both operands to
bf16, accumulates in fp32 and returns bf16; every norm is taken in fp32; pointwise ops follow
ordinary type promotion.  `Numerics(autocast=False)` is the reference on CPU: no casts except
Newton-Schulz's own `G.bfloat16()`.  `ns_dtype=None` keeps Newton-Schulz in the input dtype
(used with float64 inputs for the closed-form pins in tests/).

Parity pins (tests/test_oracle_pins.py): apply == textbook SwiGLU MLP; fast-weight gradients ==
autograd gradient of sum_t lr_t <f_w(k_t), v_t> per weight; silu_backprop == autograd of silu;
Newton-Schulz: scalar polynomial on orthogonal input, scale invariance, transpose equivariance,
SVD singular-vector preservation; momentum == unrolled recurrence; renorm row-norm identity;
schedule: update count, L<=C degenerate case, block causality.  The one statement only a run of
the reference could pin against a mis-reading is the bidirectional Muon assignment
(bidirectional_lact_layer.py:139-146); see tests/golden/.
"""
from __future__ import annotations

import collections
import math
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

# ttt_operation.py:51-57
NS5_COEFFS = (
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)
# lact_ttt.py:51, functions.py:56
NS_CLASSIC = (3.4445, -4.7750, 2.0315)

UPDATE, APPLY = 0, 1
# (kind, start, end): UPDATE consumes k,v,lr,momentum[start:end]; APPLY consumes q[start:end].
Step = collections.namedtuple("Step", ["kind", "start", "end"])
TTTOperator = collections.namedtuple("TTTOperator", ["start", "end", "update", "apply"])  # lact_ttt.py:10


@dataclass(frozen=True)
class Numerics:
    autocast: bool = False
    ns_dtype: Optional[torch.dtype] = torch.bfloat16
    # How a bf16 GEMM accumulates.  Every choice rounds at the same points (bf16 operands, bf16 result); only the
    # order / width of the additions in between differs, as it does between any two GEMM libraries:
    #   "fp32"    one fp32 matmul (the CPU library's own blocking)
    #   "fp64"    float64 accumulation
    #   "kblockN"  fp32 partial products over N consecutive k, added in ascending order (N = 16: what a
    #             matrix-core instruction with K = 16 does)
    #   "kblockNr" the same, added in descending order
    # tests/ use the spread between these ("order-only floor") as the yardstick for the Muon path, where
    # Newton-Schulz amplifies single bf16 rounding flips to percent level.
    accumulate: str = "fp32"

    def _ordered_mm(self, a: torch.Tensor, b: torch.Tensor, out_dtype) -> torch.Tensor:
        """a @ b on fp32 values with the accumulation order named by `accumulate`, result cast to out_dtype."""
        if self.accumulate == "fp32":
            return torch.matmul(a.float(), b.float()).to(out_dtype)
        if self.accumulate == "fp64":
            return torch.matmul(a.double(), b.double()).to(out_dtype)
        blk = int(self.accumulate[len("kblock"):].rstrip("r"))
        af, bfl = a.float(), b.float()
        starts = list(range(0, af.shape[-1], blk))
        if self.accumulate.endswith("r"):
            starts.reverse()
        acc = None
        for s0 in starts:
            part = torch.matmul(af[..., s0:s0 + blk], bfl[..., s0:s0 + blk, :])
            acc = part if acc is None else acc + part
        return acc.to(out_dtype)

    def mm(self, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        """Batched matmul with the autocast policy of `aten::bmm` (lower-precision list)."""
        if self.autocast:
            # bf16-rounded operands, fp32 accumulation, bf16 result (what a GPU bf16 GEMM does);
            # done as an fp32 GEMM on rounded values so that the CPU run is fast and deterministic.
            return self._ordered_mm(a.bfloat16(), b.bfloat16(), torch.bfloat16)
        if self.accumulate != "fp32" and a.dtype == b.dtype and a.dtype in (torch.bfloat16, torch.float32):
            return self._ordered_mm(a, b, a.dtype)     # no autocast: a bf16 (Newton-Schulz) or fp32 GEMM, reordered
        return torch.matmul(a, b)

    def norm(self, x: torch.Tensor, dim, keepdim=True) -> torch.Tensor:
        """Autocast keeps norms in fp32 (ttt_operation.py:26 "norm will upcast to float32").  The accumulation
        variants change the order / width of the sum of squares too (the result moves by an ulp or so)."""
        xf = x.float() if self.autocast else x
        if self.accumulate == "fp32" or xf.dtype == torch.float64:
            return xf.norm(dim=dim, keepdim=keepdim)
        out_dtype = xf.dtype
        dims = (dim,) if isinstance(dim, int) else tuple(dim)
        sq = xf.double() ** 2
        if self.accumulate == "fp64":
            ss = sq.sum(dim=dims, keepdim=keepdim)
            return ss.sqrt().float().to(out_dtype)
        # fp32 partial sums over blocks of consecutive elements, added in ascending / descending order
        blk = int(self.accumulate[len("kblock"):].rstrip("r")) * 8
        dims = tuple(d % x.dim() for d in dims)
        keep = [d for d in range(x.dim()) if d not in dims]
        flat = xf.float().permute(*keep, *dims).reshape(*[x.shape[d] for d in keep], -1)
        flat = flat * flat
        starts = list(range(0, flat.shape[-1], blk))
        if self.accumulate.endswith("r"):
            starts.reverse()
        acc = None
        for s0 in starts:
            part = flat[..., s0:s0 + blk].sum(dim=-1)
            acc = part if acc is None else acc + part
        n = acc.sqrt()
        if keepdim:
            for d in sorted(dims):
                n = n.unsqueeze(d)
        return n.to(out_dtype)


# ---------------------------------------------------------------------------------------------
# helpers (a8, a9)
# ---------------------------------------------------------------------------------------------
def silu_backprop(dy: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """ttt_operation.py:5-17: dy * s * (1 + x (1 - s)), s = sigmoid(x)."""
    s = torch.sigmoid(x)
    return dy * s * (1 + x * (1 - s))


def l2_norm(x: torch.Tensor, num: Numerics = Numerics()) -> torch.Tensor:
    """ttt_operation.py:20-27."""
    return (x / (num.norm(x, dim=-1) + 1e-5)).type(x.dtype)


def inv_softplus(x):
    """bidirectional_lact_layer.py:163-168."""
    if isinstance(x, torch.Tensor):
        return x + torch.log(-torch.expm1(-x))
    return x + math.log(-math.expm1(-x))


# ---------------------------------------------------------------------------------------------
# Newton-Schulz (a7)
# ---------------------------------------------------------------------------------------------
def ns_coeff_table(kind: str, steps: int) -> Tuple[Tuple[float, float, float], ...]:
    if kind == "llm":  # fixed 5-entry schedule, ttt_operation.py:51-57
        return NS5_COEFFS
    if kind == "classic":  # one triple repeated `steps` times, lact_ttt.py:51,58
        return tuple(NS_CLASSIC for _ in range(steps))
    raise ValueError(kind)


def newton_schulz(G: torch.Tensor, coeffs: Sequence[Tuple[float, float, float]] = NS5_COEFFS,
                  num: Numerics = Numerics()) -> torch.Tensor:
    """ttt_operation.py:30-66 / lact_ttt.py:33-67.  G: [b, m, n]."""
    assert G.dim() == 3
    X = G if num.ns_dtype is None else G.to(num.ns_dtype)
    tall = G.size(1) > G.size(2)
    if tall:
        X = X.transpose(1, 2)
    X = X / (num.norm(X, dim=(1, 2)) + 1e-7)
    for a, b, c in coeffs:
        A = num.mm(X, X.transpose(1, 2))
        # `b * A + c * A @ A` parses as b*A + ((c*A) @ A)
        B = b * A + num.mm(c * A, A)
        X = a * X + num.mm(B, X)
    if tall:
        X = X.transpose(1, 2)
    return X


# ---------------------------------------------------------------------------------------------
# stages
# ---------------------------------------------------------------------------------------------
def swiglu_apply(w0, w1, w2, q, num: Numerics = Numerics()) -> torch.Tensor:
    """ttt_operation.py:141-144.  q: [b, l, dk] -> o: [b, l, dv]."""
    qt = q.transpose(1, 2)
    h = num.mm(w2, qt)
    gate = F.silu(num.mm(w0, qt))
    return num.mm(w1, gate * h).transpose(1, 2)


def fast_weight_grads(w0, w1, w2, k, v, lr0, lr1, lr2, num: Numerics = Numerics(),
                      cast_lr_operand: bool = True, w_scale: Optional[float] = None):
    """ttt_operation.py:147-168.  Returns (dw0, dw1, dw2), the lr-weighted descent direction of
    L = -sum_t <f_w(k_t), v_t>.  `cast_lr_operand=False` is the AR-video spelling
    (ar_lact_swa_repeat.py:134-138), which leaves the lr-scaled operand in fp32 until the matmul and
    multiplies by `w_scale` AFTER the learning rate: (k * lr) * w_scale."""
    kt = k.transpose(1, 2)          # [b, dk, l]
    vt = v.transpose(1, 2)          # [b, dv, l]
    g = num.mm(w0, kt)              # gate_before_act   [b, dh, l]
    h2 = num.mm(w2, kt)             # hidden_before_mul
    sg = F.silu(g)
    hidden = sg * h2
    dh = num.mm(w1.transpose(1, 2), vt)
    dh2 = dh * sg
    dg = silu_backprop(dh * h2, g)
    r1 = hidden.transpose(1, 2) * lr1
    r0 = k * lr0
    r2 = k * lr2
    if w_scale is not None:         # ar_lact_swa_repeat.py:134-138: left to right, the scale last
        r1, r0, r2 = r1 * w_scale, r0 * w_scale, r2 * w_scale
    if cast_lr_operand:
        r1, r0, r2 = r1.type_as(vt), r0.type_as(dg), r2.type_as(dh2)
    dw1 = num.mm(vt, r1)
    dw0 = num.mm(dg, r0)
    dw2 = num.mm(dh2, r2)
    return dw0, dw1, dw2


def renorm(w: torch.Tensor, w_norm0: torch.Tensor, num: Numerics = Numerics(), eps_in_sqrt: bool = False) -> torch.Tensor:
    """ttt_operation.py:198-200: rows rescaled to their initial L2 norm, eps outside the sqrt.
    eps_in_sqrt: the fused variant's kernel (l2norm_triton_kernels.py:205-214, "eps is inside the sqrt"):
    y = x / sqrt(sum(x^2) + eps) * scale, statistics in fp32."""
    if eps_in_sqrt:
        wf = w.float()
        rstd = torch.rsqrt((wf * wf).sum(dim=2, keepdim=True) + 1e-5)
        return (wf * rstd * w_norm0.float()).to(w.dtype)
    return w / (num.norm(w, dim=2) + 1e-5) * w_norm0


# ---------------------------------------------------------------------------------------------
# the interpreter
# ---------------------------------------------------------------------------------------------
def run_program(w0, w1, w2, q, k, v, lr0, lr1, lr2, steps: Sequence[Step], *,
                num: Numerics = Numerics(),
                ns_coeffs: Optional[Sequence[Tuple[float, float, float]]] = None,
                momentum: Optional[torch.Tensor] = None,
                prenorm: bool = False,
                weight_norm: bool = True,
                detach_norms: bool = False,
                muon_replaces_weight: bool = False,
                cast_lr_operand: bool = True,
                out_rows: Optional[int] = None,
                scatter_output: bool = True,
                w_scale: Optional[float] = None,
                stack_muon: bool = False,
                eps_in_sqrt: bool = False,
                momentum_state: Optional[Sequence[torch.Tensor]] = None):
    """Runs UPDATE / APPLY steps over one sequence.  LLM layout: w0,w2 [b,dh,dk], w1 [b,dv,dh].

    ns_coeffs=None means no Muon.  `muon_replaces_weight` is the bidirectional layer's behaviour
    (bidirectional_lact_layer.py:139-146): the orthogonalised gradient overwrites the weight and
    the raw gradient is then added, w_hat = NS(dw) + dw.
    `stack_muon` / `eps_in_sqrt` are the two places where the fused-kernel driver differs in semantics
    (ttt_operation_fused_kernel.py:106,168-173): Newton-Schulz runs on the stacked gradient cat(dw0, dw2)
    [b, 2dh, d] (one Frobenius norm, one orthogonalisation) and the row renorm has eps inside the sqrt.
    Returns (output, (w0, w1, w2), (m0, m1, m2) or None).
    """
    def init_norm(w):
        w_ = w.detach() if detach_norms else w
        return num.norm(w_, dim=2)
    n0, n1, n2 = init_norm(w0), init_norm(w1), init_norm(w2)
    main0, main1, main2 = w0, w1, w2               # ttt_operation.py:260 (pre-norm accumulator)
    mom = None
    if momentum is not None:                        # ttt_operation.py:112-115
        mom = [torch.zeros_like(w0), torch.zeros_like(w1), torch.zeros_like(w2)]
        if momentum_state is not None:              # ar_lact_swa_repeat_sp.py:266-269 (state carried between calls)
            mom = list(momentum_state)

    pieces: List[Tuple[int, int, torch.Tensor]] = []
    for kind, s, e in steps:
        if kind == APPLY:
            pieces.append((s, e, swiglu_apply(w0, w1, w2, q[:, s:e], num)))
            continue
        dw0, dw1, dw2 = fast_weight_grads(w0, w1, w2, k[:, s:e], v[:, s:e],
                                          lr0[:, s:e], lr1[:, s:e], lr2[:, s:e], num,
                                          cast_lr_operand, w_scale)
        if mom is not None:                         # ttt_operation.py:170-179
            m = momentum[:, s:e].mean(dim=1, keepdim=True)
            dw0 = dw0 + mom[0] * m
            dw1 = dw1 + mom[1] * m
            dw2 = dw2 + mom[2] * m
            mom = [dw0, dw1, dw2]
        raw = (dw0, dw1, dw2)
        if ns_coeffs is not None and stack_muon:    # ttt_operation_fused_kernel.py:168-170
            dw1 = newton_schulz(dw1, ns_coeffs, num)
            stacked = newton_schulz(torch.cat([dw0, dw2], dim=1), ns_coeffs, num)
            dw0, dw2 = stacked[:, :dw0.shape[1]], stacked[:, dw0.shape[1]:]
        elif ns_coeffs is not None:                 # ttt_operation.py:181-184
            dw1 = newton_schulz(dw1, ns_coeffs, num)
            dw0 = newton_schulz(dw0, ns_coeffs, num)
            dw2 = newton_schulz(dw2, ns_coeffs, num)
        if muon_replaces_weight and ns_coeffs is not None:
            main0, main1, main2 = dw0 + raw[0], dw1 + raw[1], dw2 + raw[2]
        else:                                       # ttt_operation.py:193-195 / :343-345
            base = (main0, main1, main2) if prenorm else (w0, w1, w2)
            main0, main1, main2 = base[0] + dw0, base[1] + dw1, base[2] + dw2
        if weight_norm:                             # ttt_operation.py:198-200 / :348-350
            w0, w1, w2 = (renorm(main0, n0, num, eps_in_sqrt), renorm(main1, n1, num, eps_in_sqrt),
                          renorm(main2, n2, num, eps_in_sqrt))
        else:
            w0, w1, w2 = main0, main1, main2

    if not pieces:
        out = None
    elif scatter_output:                            # ttt_operation.py:119,144,212
        rows = out_rows if out_rows is not None else q.shape[1]
        out = torch.zeros(q.shape[0], rows, w1.shape[1], dtype=pieces[0][2].dtype, device=q.device)
        # later writes win, as with the reference's slice assignment
        out = _assemble(out, pieces)
    else:                                           # lact_ttt.py:142-145 (concatenate in program order)
        out = torch.cat([o for _, _, o in pieces], dim=1)
    return out, (w0, w1, w2), (tuple(mom) if mom is not None else None)


def _assemble(buf: torch.Tensor, pieces):
    """Slice-assign each piece into buf in order (autograd tracks overwritten rows correctly)."""
    out = buf
    for s, e, o in pieces:
        out = torch.cat([out[:, :s], o.to(out.dtype), out[:, e:]], dim=1)
    return out


# ---------------------------------------------------------------------------------------------
# schedules
# ---------------------------------------------------------------------------------------------
def block_causal_steps(seq_len: int, chunk_size: int) -> List[Step]:
    """ttt_operation.py:121-212: apply chunk i with the weights of chunks < i, then update on
    chunk i; the last (possibly ragged, possibly whole-sequence) chunk is apply-only."""
    steps: List[Step] = []
    e = 0
    for s in range(0, seq_len - chunk_size, chunk_size):
        e = s + chunk_size
        steps.append(Step(APPLY, s, e))
        steps.append(Step(UPDATE, s, e))
    steps.append(Step(APPLY, e, seq_len))
    return steps


def ar_video_steps(seq_len: int, mini_batch_size: int, update_length: int, update_every: int,
                   num_repeat: int = 1) -> List[Step]:
    """ar_lact_swa_repeat.py:76-165: clean/noisy interleave, update on the clean chunk then apply
    on clean+noisy."""
    if update_length == -1:
        update_length = seq_len
    if mini_batch_size == -1:
        mini_batch_size = update_length
    if update_every == -1:
        update_every = mini_batch_size * 2
    first = update_every - mini_batch_size
    steps = [Step(APPLY, 0, first)]
    for _ in range(num_repeat):
        for s in range(first, update_length, update_every):
            steps.append(Step(UPDATE, s, s + mini_batch_size))
            steps.append(Step(APPLY, s, min(s + update_every, seq_len)))
    return steps


# ---------------------------------------------------------------------------------------------
# entry points with the reference's names and argument orders
# ---------------------------------------------------------------------------------------------
def block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size: int = 2048,
                             use_muon: bool = False, momentum: Optional[torch.Tensor] = None, *,
                             num: Numerics = Numerics(), prenorm: bool = False):
    """ttt_operation.py:71-214 (prenorm=True: :219-364)."""
    out, _, _ = run_program(w0, w1, w2, q, k, v, lr0, lr1, lr2,
                            block_causal_steps(k.shape[1], chunk_size), num=num,
                            ns_coeffs=NS5_COEFFS if use_muon else None,
                            momentum=momentum, prenorm=prenorm)
    return out


def prenorm_block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size: int = 2048,
                                     use_muon: bool = False, momentum=None, *,
                                     num: Numerics = Numerics()):
    """ttt_operation.py:219-364."""
    return block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon,
                                    momentum, num=num, prenorm=True)


def postnorm_block_causal_lact_swiglu_fused_kernel_triton(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size: int = 2048,
                                                          use_muon: bool = False, momentum=None, *,
                                                          num: Numerics = Numerics()):
    """ttt_operation_fused_kernel.py:67-199: the schedule of block_causal_lact_swiglu (padding to whole chunks
    changes nothing: only whole chunks update), Muon on the stacked cat(dw0, dw2), eps inside the sqrt."""
    out, _, _ = run_program(w0, w1, w2, q, k, v, lr0, lr1, lr2,
                            block_causal_steps(k.shape[1], chunk_size), num=num,
                            ns_coeffs=NS5_COEFFS if use_muon else None, momentum=momentum,
                            stack_muon=True, eps_in_sqrt=True)
    return out


def prenorm_block_causal_lact_swiglu_fused_kernel_triton(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size: int = 2048,
                                                         use_muon: bool = False, momentum=None, *,
                                                         num: Numerics = Numerics()):
    """ttt_operation_fused_kernel.py:202-338: pre-norm accumulator, Muon on the stacked gradient, eps outside
    the sqrt (:322-327)."""
    out, _, _ = run_program(w0, w1, w2, q, k, v, lr0, lr1, lr2,
                            block_causal_steps(k.shape[1], chunk_size), num=num,
                            ns_coeffs=NS5_COEFFS if use_muon else None, momentum=momentum, prenorm=True,
                            stack_muon=True)
    return out


def block_causal_lact_swiglu_minimal(w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum=None,
                                     use_muon: bool = True, chunk_size: int = 2048, *,
                                     num: Numerics = Numerics()):
    """causal_lact_with_sliding_window_attn.py:84-211 (argument order :94-96)."""
    return block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon,
                                    momentum, num=num)


def bidirectional_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, use_muon: bool = True, *,
                              num: Numerics = Numerics(), muon_mode: str = "reference"):
    """bidirectional_lact_layer.py:74-160.  muon_mode="reference" keeps the layer's assignment
    w = NS(dw); w = w + dw  (:139-146); "intended" does w + NS(dw) like every other variant."""
    L = k.shape[1]
    out, _, _ = run_program(w0, w1, w2, q, k, v, lr0, lr1, lr2,
                            [Step(UPDATE, 0, L), Step(APPLY, 0, q.shape[1])], num=num,
                            ns_coeffs=NS5_COEFFS if use_muon else None,
                            muon_replaces_weight=(muon_mode == "reference"))
    return out


def fast_weight_swish_glu_weight_norm_mini_batch_apply(w0, w1, w2, q, k, v, lr0, lr1, lr2,
                                                       ttt_ua_order, muon_update_steps: int = 0, *,
                                                       num: Numerics = Numerics()):
    """lact_nvs/lact_ttt.py:71-147.  Transposed layout: w0,w2 [b,d,dh], w1 [b,dh,d]; norms over
    dim=1 and detached (:96-98); Newton-Schulz always runs (steps=0 is cast + Frobenius
    normalisation only); an operator with update and apply applies the *updated* weights (:140-143)."""
    steps: List[Step] = []
    for start, end, update, apply in ttt_ua_order:
        if update:
            steps.append(Step(UPDATE, start, end))
        if apply:
            steps.append(Step(APPLY, start, end))
    out, (a0, a1, a2), _ = run_program(
        w0.transpose(1, 2), w1.transpose(1, 2), w2.transpose(1, 2), q, k, v, lr0, lr1, lr2, steps,
        num=num, ns_coeffs=ns_coeff_table("classic", muon_update_steps), detach_norms=True,
        cast_lr_operand=False, scatter_output=False)
    return out, a0.transpose(1, 2), a1.transpose(1, 2), a2.transpose(1, 2)


def ar_fast_weight_swish_glu_weight_norm_mini_batch(w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale: float,
                                                    num_repeat: int = 1, mini_batch_size: int = -1,
                                                    update_length: int = -1, update_every: int = -1,
                                                    use_moun: bool = False, num_moun_iters: int = 3,
                                                    weight_norm: bool = True,
                                                    fw_momentum: Optional[torch.Tensor] = None,
                                                    use_momentum: bool = False, *,
                                                    num: Numerics = Numerics()):
    """ar_lact_swa_repeat.py:23-168 and, with momentum, ar_lact_swa_repeat_sp.py:28-193."""
    steps = ar_video_steps(k.shape[1], mini_batch_size, update_length, update_every, num_repeat)
    out, ws, _ = run_program(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, steps, num=num, w_scale=w_scale,
        ns_coeffs=ns_coeff_table("classic", num_moun_iters) if use_moun else None,
        momentum=fw_momentum if use_momentum else None, weight_norm=weight_norm,
        cast_lr_operand=False)
    return (out,) + tuple(ws)


def ar_fast_weight_swish_glu_weight_norm_mini_batch_inference(w0, w1, w2, q, k, v, lr0, lr1, lr2,
                                                              w_scale: float, num_repeat: int = 1,
                                                              mini_batch_size: int = -1,
                                                              do_update: bool = False,
                                                              use_moun: bool = False,
                                                              num_moun_iters: int = 3,
                                                              weight_norm: bool = True, *,
                                                              num: Numerics = Numerics()):
    """ar_lact_swa_repeat.py:172-296: optional repeated update on k,v[:mini_batch] then apply on all q."""
    mb = k.shape[1] if mini_batch_size == -1 else mini_batch_size
    steps = [Step(UPDATE, 0, mb) for _ in range(num_repeat)] if do_update else []
    steps.append(Step(APPLY, 0, q.shape[1]))
    out, ws, _ = run_program(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, steps, num=num, w_scale=w_scale,
        ns_coeffs=ns_coeff_table("classic", num_moun_iters) if use_moun else None,
        weight_norm=weight_norm, cast_lr_operand=False)
    return (out,) + tuple(ws)


def ar_fast_weight_swish_glu_weight_norm_mini_batch_inference_with_momentum(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale: float, num_repeat: int = 1, mini_batch_size: int = -1,
        do_update: bool = False, use_moun: bool = False, num_moun_iters: int = 3, weight_norm: bool = True,
        fw_momentum: Optional[torch.Tensor] = None, dw0_momentum=None, dw1_momentum=None, dw2_momentum=None,
        use_momentum: bool = False, *, num: Numerics = Numerics()):
    """ar_lact_swa_repeat_sp.py:197-339: the inference step whose momentum states travel between calls.
    Returns (output, w0, w1, w2, m0, m1, m2); the states come back untouched when no update runs, as zeros when
    momentum is on and none were given (:266-269), and as None when momentum is off."""
    mb = k.shape[1] if mini_batch_size == -1 else mini_batch_size
    steps = [Step(UPDATE, 0, mb) for _ in range(num_repeat)] if do_update else []
    steps.append(Step(APPLY, 0, q.shape[1]))
    state = None
    if use_momentum:
        state = ((dw0_momentum, dw1_momentum, dw2_momentum) if dw0_momentum is not None
                 else (torch.zeros_like(w0), torch.zeros_like(w1), torch.zeros_like(w2)))
    out, ws, ms = run_program(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, steps, num=num, w_scale=w_scale,
        ns_coeffs=ns_coeff_table("classic", num_moun_iters) if use_moun else None,
        momentum=fw_momentum if use_momentum else None, weight_norm=weight_norm,
        cast_lr_operand=False, momentum_state=state)
    if not use_momentum:
        ms = (dw0_momentum, dw1_momentum, dw2_momentum)
    return (out,) + tuple(ws) + tuple(ms)


# ---------------------------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations (seeded, generated on the CPU in fp32)
# ---------------------------------------------------------------------------------------------
def make_inputs(b: int, L: int, d: int, dh: int, *, seed: int, act_dtype=torch.bfloat16,
                lr_shift: float = -3.0, lr_scale: float = 1.0, momentum_value: Optional[float] = 0.9,
                distinct_heads: Optional[int] = None, normalize_v: bool = False):
    """q,k ~ N(0,1) L2-normalised per token, v ~ N(0,1); w0,w2 ~ N(0,1)/sqrt(d), w1 ~ N(0,1)/sqrt(dh)
    (layer_lact_swiglu.py:214-222), optionally `distinct_heads` matrices repeated over the batch
    (:452-461); lr = softplus(N(0,1)+lr_shift)*lr_scale; momentum constant."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    q, k, v = rn(b, L, d), rn(b, L, d), rn(b, L, d)
    q = q / (q.norm(dim=-1, keepdim=True) + 1e-5)
    k = k / (k.norm(dim=-1, keepdim=True) + 1e-5)
    if normalize_v:
        v = v / (v.norm(dim=-1, keepdim=True) + 1e-5)
    nh = distinct_heads or b
    w0 = (rn(nh, dh, d) / math.sqrt(d)).repeat(b // nh, 1, 1)
    w2 = (rn(nh, dh, d) / math.sqrt(d)).repeat(b // nh, 1, 1)
    w1 = (rn(nh, d, dh) / math.sqrt(dh)).repeat(b // nh, 1, 1)
    lr0, lr1, lr2 = (F.softplus(rn(b, L, 1) + lr_shift) * lr_scale for _ in range(3))
    mom = None if momentum_value is None else torch.full((b, L, 1), float(momentum_value))
    return dict(w0=w0, w1=w1, w2=w2, q=q.to(act_dtype), k=k.to(act_dtype), v=v.to(act_dtype),
                lr0=lr0, lr1=lr1, lr2=lr2, momentum=mom)


ORDER_VARIANTS = ("fp64", "kblock16", "kblock64r")


def order_variants(num: Numerics):
    """The same numerics with each of the other accumulation orders (see Numerics.accumulate)."""
    return [Numerics(autocast=num.autocast, ns_dtype=num.ns_dtype, accumulate=a) for a in ORDER_VARIANTS]


def rel_l2(a: torch.Tensor, ref: torch.Tensor) -> float:
    a, ref = a.detach().double().cpu(), ref.detach().double().cpu()
    return float((a - ref).norm() / (ref.norm() + 1e-30))
