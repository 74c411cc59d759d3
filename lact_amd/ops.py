"""Host side of the TTT operation: turns a schedule into the C ABI's step program, owns the
autograd boundary and the buffers, and calls liblact_hip.so on the current HIP stream.

PyTorch is used for device memory, streams and autograd bookkeeping only; all arithmetic of the
operation runs in the HIP kernels.  There is no fallback path.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import LACT_APPLY, LACT_BF16, LACT_F32, LACT_UPDATE

# lact_llm/lact_model/ttt_operation.py:51-57
NS5_COEFFS: Tuple[Tuple[float, float, float], ...] = (
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)
# lact_nvs/lact_ttt.py:51 and lact_ar_video/minVid/models/blocks/functions.py:56
NS_CLASSIC: Tuple[float, float, float] = (3.4445, -4.7750, 2.0315)


@dataclass(frozen=True)
class Program:
    """A test-time-training schedule: steps are (kind, start, end, out_start)."""
    steps: Tuple[Tuple[int, int, int, int], ...]
    out_len: int
    ns_coeffs: Optional[Tuple[Tuple[float, float, float], ...]] = None   # None: Muon off
    prenorm: bool = False
    weight_norm: bool = True
    detach_norms: bool = False
    muon_replaces_weight: bool = False
    ns_mode: int = 0   # 0: bf16 GEMMs + fp32 iterate (autocast), 1: bf16 iterate (no autocast), 2: fp32 (exact)
    # fused-kernel variant (lact_llm/lact_model/ttt_operation_fused_kernel.py): Newton-Schulz on the stacked
    # gradient cat(dw0, dw2); eps inside the sqrt of the row renorm
    muon_stacked: bool = False
    renorm_eps_in_sqrt: bool = False
    # callers that only use the output (the block-causal and bidirectional functions) spare the copies of the final
    # fast weights and momentum states: run_program then returns None in their places
    return_state: bool = True

    @property
    def n_updates(self) -> int:
        return sum(1 for s in self.steps if s[0] == LACT_UPDATE)


def block_causal_steps(seq_len: int, chunk_size: int):
    """Apply chunk i with the weights of chunks < i, then update on chunk i; the last chunk is
    apply-only (lact_llm/lact_model/ttt_operation.py:121-212)."""
    steps, e = [], 0
    for s in range(0, seq_len - chunk_size, chunk_size):
        e = s + chunk_size
        steps.append((LACT_APPLY, s, e, s))
        steps.append((LACT_UPDATE, s, e, 0))
    steps.append((LACT_APPLY, e, seq_len, e))
    return tuple(steps)


def _rows_view(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """[b, L, d] tensor whose rows the kernels can read with 16-byte vectors."""
    if t.dtype != dtype:
        t = t.to(dtype)
    align = 16 // t.element_size()
    ok = (t.dim() == 3 and t.stride(2) == 1 and t.stride(1) % align == 0 and t.stride(0) % align == 0
          and t.stride(1) >= t.shape[2] and t.data_ptr() % 16 == 0)
    return t if ok else t.contiguous()


def _per_token(t: torch.Tensor, b: int, L: int, name: str) -> torch.Tensor:
    if t.numel() != b * L:
        raise ValueError(f"{name} must hold one value per head and token ([b, l, 1]); got {tuple(t.shape)}")
    return t.reshape(b, L).float().contiguous()


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _ptr3(ts: Sequence[Optional[torch.Tensor]]):
    arr = (ctypes.c_void_p * 3)(*[0 if t is None else t.data_ptr() for t in ts])
    return arr


class _Call:
    """Descriptor plus the Python objects that must outlive the C call."""

    def __init__(self, prog: Program, b, d, dh, q, k, v, out, dout=None):
        self.steps = (_lib.Step * len(prog.steps))(*[_lib.Step(*s) for s in prog.steps])
        ns = prog.ns_coeffs
        self.coeffs = None
        if ns is not None and len(ns) > 0:
            flat = [float(x) for tr in ns for x in tr]
            self.coeffs = (ctypes.c_float * len(flat))(*flat)
        D = _lib.Desc()
        D.b, D.d, D.dh = b, d, dh
        D.q_len, D.kv_len, D.out_len = q.shape[1], (k.shape[1] if k is not None else 0), prog.out_len
        D.act_dtype = LACT_BF16 if q.dtype == torch.bfloat16 else LACT_F32
        D.n_steps = len(prog.steps)
        D.steps = ctypes.cast(self.steps, ctypes.POINTER(_lib.Step))
        D.ns_steps = -1 if ns is None else len(ns)
        D.ns_coeffs = ctypes.cast(self.coeffs, ctypes.POINTER(ctypes.c_float)) if self.coeffs is not None else None
        D.use_momentum = 0
        D.prenorm, D.weight_norm = int(prog.prenorm), int(prog.weight_norm)
        D.detach_norms, D.muon_replaces_weight = int(prog.detach_norms), int(prog.muon_replaces_weight)
        D.ns_mode = int(prog.ns_mode)
        D.muon_stacked, D.renorm_eps_in_sqrt = int(prog.muon_stacked), int(prog.renorm_eps_in_sqrt)
        D.q_bs, D.q_ld = q.stride(0), q.stride(1)
        if k is not None:
            D.k_bs, D.k_ld, D.v_bs, D.v_ld = k.stride(0), k.stride(1), v.stride(0), v.stride(1)
        else:
            D.k_bs, D.k_ld, D.v_bs, D.v_ld = 0, d, 0, d
        D.o_bs, D.o_ld = out.stride(0), out.stride(1)
        if dout is not None:
            D.do_bs, D.do_ld = dout.stride(0), dout.stride(1)
        else:
            D.do_bs, D.do_ld = out.stride(0), out.stride(1)
        self.desc = D

    def sizes(self) -> Tuple[int, int]:
        a, b = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _lib.check(_lib.lib().lact_query_sizes(ctypes.byref(self.desc), ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value


def _covers(steps, out_len: int) -> bool:
    iv = sorted((s[3], s[3] + s[2] - s[1]) for s in steps if s[0] == LACT_APPLY)
    pos = 0
    for a, e in iv:
        if a > pos:
            return False
        pos = max(pos, e)
    return pos >= out_len


class _LactProgramFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, prog: Program, w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum, m_state=None, grad_mode=True):
        if not q.is_cuda:
            raise RuntimeError("lact_amd runs on an MI355X only: tensors must be on a HIP device (no CPU path)")
        L = _lib.lib()
        b, dh, d = w0.shape
        if w1.shape != (b, d, dh) or w2.shape != (b, dh, d):
            raise ValueError("expected w0, w2: [b, dh, d] and w1: [b, d, dh] with equal key and value dims")
        act = torch.bfloat16 if q.dtype in (torch.bfloat16, torch.float16) else torch.float32
        if torch.is_autocast_enabled():
            act = torch.bfloat16
        qa = _rows_view(q, act)
        has_update = prog.n_updates > 0
        ka = _rows_view(k, act) if has_update else None
        va = _rows_view(v, act) if has_update else None
        kv_len = ka.shape[1] if has_update else 0
        wf = [w.detach().float().contiguous() for w in (w0, w1, w2)]
        lrs = [_per_token(t, b, kv_len, "lr") if has_update else None for t in (lr0, lr1, lr2)]
        mom = _per_token(momentum, b, kv_len, "momentum") if (momentum is not None and has_update) else None
        alloc = torch.empty if _covers(prog.steps, prog.out_len) else torch.zeros
        out = alloc((b, prog.out_len, d), dtype=act, device=q.device)
        call = _Call(prog, b, d, dh, qa, ka, va, out)
        call.desc.use_momentum = int(mom is not None)
        # needs_input_grad ignores the grad mode (and inside forward grad mode is always off): the caller's mode
        # comes in as an argument -- under torch.no_grad() nothing will ask for a backward pass
        call.desc.forward_only = int(not (grad_mode and any(ctx.needs_input_grad)))
        m_in = None
        if m_state is not None and mom is not None:
            if not call.desc.forward_only:
                raise RuntimeError("a carried momentum state is an inference feature: call under torch.no_grad()")
            m_in = [m.detach().float().contiguous() for m in m_state]
            if any(m.shape != w.shape for m, w in zip(m_in, wf)):
                raise ValueError("momentum states must have the shapes of w0, w1, w2")
            call.desc.momentum_state_in = 1
        saved_bytes, scratch_bytes = call.sizes()
        saved = torch.empty(saved_bytes, dtype=torch.uint8, device=q.device)
        scratch = torch.empty(scratch_bytes, dtype=torch.uint8, device=q.device)
        w_out = [torch.empty_like(w) for w in wf] if prog.return_state else [None, None, None]
        m_out = [torch.empty_like(w) for w in wf] if (mom is not None and prog.return_state) else [None, None, None]
        stream = ctypes.c_void_p(torch.cuda.current_stream(q.device).cuda_stream)
        with torch.cuda.device(q.device):
            _lib.check(L.lact_forward_from_state(
                ctypes.byref(call.desc), _ptr(wf[0]), _ptr(wf[1]), _ptr(wf[2]), _ptr(qa), _ptr(ka), _ptr(va), _ptr(lrs[0]),
                _ptr(lrs[1]), _ptr(lrs[2]), _ptr(mom), None if m_in is None else _ptr3(m_in), _ptr(out), _ptr3(w_out),
                _ptr3(m_out), _ptr(saved), _ptr(scratch), stream))
        ctx.prog, ctx.dims = prog, (b, d, dh)
        ctx.in_dtypes = (w0.dtype, w1.dtype, w2.dtype, q.dtype, k.dtype if k is not None else None,
                         v.dtype if v is not None else None)
        ctx.shapes = (lr0.shape if lr0 is not None else None, momentum.shape if momentum is not None else None)
        ctx.lr_dtype = lr0.dtype if lr0 is not None else torch.float32
        ctx.mom_dtype = momentum.dtype if momentum is not None else None
        ctx.save_for_backward(qa, ka, va, lrs[0], lrs[1], lrs[2], mom, saved)
        ctx.mark_non_differentiable(*[m for m in m_out if m is not None])
        ctx.set_materialize_grads(False)   # unused outputs arrive as None in backward, not as zero tensors
        out_dtype = q.dtype if q.dtype in (torch.bfloat16, torch.float32) else act
        if v is not None and v.dtype == torch.float32 and act == torch.bfloat16:
            out_dtype = torch.float32          # zeros_like(v) receives the bf16 products
        res_out = out if out.dtype == out_dtype else out.to(out_dtype)
        if not prog.return_state:
            return (res_out, None, None, None, None, None, None)
        return (res_out, w_out[0], w_out[1], w_out[2]) + tuple(m_out)   # no momentum: no states (None), not zero tensors

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, g_out, g_w0, g_w1, g_w2, *_unused):
        qa, ka, va, lr0, lr1, lr2, mom, saved = ctx.saved_tensors
        prog = ctx.prog
        b, d, dh = ctx.dims
        L = _lib.lib()
        dev, act = qa.device, qa.dtype
        if g_out is None:
            g_out = torch.zeros((b, prog.out_len, d), dtype=act, device=dev)
        g_out = _rows_view(g_out, act)
        has_update = prog.n_updates > 0
        kv_len = ka.shape[1] if has_update else 0
        gwf = [None if g is None else g.float().contiguous() for g in (g_w0, g_w1, g_w2)]
        call = _Call(prog, b, d, dh, qa, ka, va, g_out, dout=g_out)
        call.desc.use_momentum = int(mom is not None)
        _, scratch_bytes = call.sizes()
        scratch = torch.empty(scratch_bytes, dtype=torch.uint8, device=dev)
        dw = [torch.empty((b, dh, d), dtype=torch.float32, device=dev),
              torch.empty((b, d, dh), dtype=torch.float32, device=dev),
              torch.empty((b, dh, d), dtype=torch.float32, device=dev)]
        # lact_backward writes every element of its outputs (rows no step touches are zeroed by the library)
        dq = torch.empty((b, qa.shape[1], d), dtype=act, device=dev)
        dk = torch.empty((b, kv_len, d), dtype=act, device=dev) if has_update else None
        dv = torch.empty((b, kv_len, d), dtype=act, device=dev) if has_update else None
        dlr = [torch.empty((b, kv_len), dtype=torch.float32, device=dev) if has_update else None for _ in range(3)]
        dmom = torch.empty((b, kv_len), dtype=torch.float32, device=dev) if mom is not None else None
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        with torch.cuda.device(dev):
            _lib.check(L.lact_backward(ctypes.byref(call.desc), _ptr(qa), _ptr(ka), _ptr(va), _ptr(lr0), _ptr(lr1),
                                       _ptr(lr2), _ptr(mom), _ptr(g_out), _ptr3(gwf), _ptr(saved), _ptr(scratch),
                                       _ptr(dw[0]), _ptr(dw[1]), _ptr(dw[2]), _ptr(dq), _ptr(dk), _ptr(dv),
                                       _ptr(dlr[0]), _ptr(dlr[1]), _ptr(dlr[2]), _ptr(dmom), stream))
        wd0, wd1, wd2, qd, kd, vd = ctx.in_dtypes
        lr_shape, mom_shape = ctx.shapes
        cast = lambda t, dt: None if t is None else (t if t.dtype == dt else t.to(dt))
        glr = [None if g is None else g.reshape(lr_shape).to(ctx.lr_dtype) for g in dlr]
        gm = None if dmom is None else dmom.reshape(mom_shape).to(ctx.mom_dtype)
        return (None, cast(dw[0], wd0), cast(dw[1], wd1), cast(dw[2], wd2), cast(dq, qd), cast(dk, kd), cast(dv, vd),
                glr[0], glr[1], glr[2], gm, None, None)


@torch.compiler.disable
def run_program(prog: Program, w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum=None, momentum_state=None):
    """Runs `prog`.  Returns (out, (w0, w1, w2) after the last update, (m0, m1, m2) momentum states; None each
    without momentum).
    `momentum_state` = the (m0, m1, m2) of an earlier call: the first update continues from it (inference only)."""
    res = _LactProgramFn.apply(prog, w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum, momentum_state, torch.is_grad_enabled())
    return res[0], res[1:4], res[4:7]


NS_AUTOCAST, NS_PLAIN_BF16, NS_FP32 = 0, 1, 2
_ns_mode_override: Optional[int] = None


class newton_schulz_mode:
    """Context manager forcing the Newton-Schulz numerics of every operation called inside it
    (NS_FP32 = fp32 MFMA, no bf16 rounding: the exact-arithmetic check of the Muon path)."""

    def __init__(self, mode: Optional[int]):
        self.mode = mode

    def __enter__(self):
        global _ns_mode_override
        self.prev, _ns_mode_override = _ns_mode_override, self.mode
        return self

    def __exit__(self, *exc):
        global _ns_mode_override
        _ns_mode_override = self.prev
        return False


def _ns_mode(q: torch.Tensor) -> int:
    """Without autocast and with fp32 activations the reference keeps the whole Newton-Schulz
    iterate in bf16 (ttt_operation.py:45 casts, nothing casts back)."""
    if _ns_mode_override is not None:
        return _ns_mode_override
    return NS_PLAIN_BF16 if (q.dtype == torch.float32 and not torch.is_autocast_enabled()) else NS_AUTOCAST


class _NewtonSchulzFn(torch.autograd.Function):
    """zeropower_via_newtonschulz5 with its closed-form backward (lact_newton_schulz / lact_newton_schulz_backward)."""

    @staticmethod
    def forward(ctx, G, coeffs, ns_mode):
        L = _lib.lib()
        n, rows, cols = G.shape
        g = G.detach().float().contiguous()
        out = torch.empty_like(g)
        ws = torch.empty(L.lact_newton_schulz_workspace_bytes(n, rows, cols, len(coeffs)), dtype=torch.uint8, device=G.device)
        flat = [float(x) for tr in coeffs for x in tr]
        arr = (ctypes.c_float * max(1, len(flat)))(*flat)
        stream = ctypes.c_void_p(torch.cuda.current_stream(G.device).cuda_stream)
        with torch.cuda.device(G.device):
            _lib.check(L.lact_newton_schulz(n, rows, cols, _ptr(g), _ptr(out), len(coeffs), arr, int(ns_mode), _ptr(ws), stream))
        ctx.save_for_backward(g)
        ctx.coeffs, ctx.ns_mode, ctx.in_dtype = tuple(coeffs), int(ns_mode), G.dtype
        return out.to(torch.bfloat16) if ns_mode == NS_PLAIN_BF16 else out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dout):
        (g,) = ctx.saved_tensors
        L = _lib.lib()
        n, rows, cols = g.shape
        do = dout.detach().float().contiguous()
        dg = torch.empty_like(g)
        steps = len(ctx.coeffs)
        ws = torch.empty(L.lact_newton_schulz_backward_workspace_bytes(n, rows, cols, steps), dtype=torch.uint8, device=g.device)
        flat = [float(x) for tr in ctx.coeffs for x in tr]
        arr = (ctypes.c_float * max(1, len(flat)))(*flat)
        stream = ctypes.c_void_p(torch.cuda.current_stream(g.device).cuda_stream)
        with torch.cuda.device(g.device):
            _lib.check(L.lact_newton_schulz_backward(n, rows, cols, _ptr(g), _ptr(do), _ptr(dg), steps, arr, ctx.ns_mode, _ptr(ws), stream))
        return dg.to(ctx.in_dtype), None, None


@torch.compiler.disable
def newton_schulz(G: torch.Tensor, coeffs: Sequence[Tuple[float, float, float]], ns_mode: int = NS_PLAIN_BF16) -> torch.Tensor:
    """zeropower_via_newtonschulz5 on [n, rows, cols] (ttt_operation.py:30-66; lact_ttt.py:33-67), differentiable."""
    if G.dim() != 3:
        raise AssertionError("expected a 3-D tensor")          # ttt_operation.py:44
    if not G.is_cuda:
        raise RuntimeError("lact_amd runs on an MI355X only (no CPU path)")
    return _NewtonSchulzFn.apply(G, tuple(tuple(c) for c in coeffs), int(ns_mode))


def check_async_error() -> None:
    """Raises if a barrier wait of the fused Newton-Schulz kernel timed out on the current device since the last check
    (the results of those steps are NaN).  Synchronises the device; call it at a point where the host waits anyway."""
    torch.cuda.synchronize()
    n = _lib.lib().lact_check_async_error()
    if n != 0:
        raise RuntimeError("liblact_hip: " + _lib.lib().lact_last_error().decode())
