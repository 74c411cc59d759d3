"""Drop-ins for the reference's layer classes around the TTT operation, with the reference's constructor
arguments and parameter names (a state_dict moves over unchanged):

  BidirectionalLaCTSwiGLU                minimal_implementations/bidirectional_lact_layer.py:171-270
  CausalLaCTSwiGLUWithSlidingWindowAttn  minimal_implementations/causal_lact_with_sliding_window_attn.py:222-391
  FastWeightGluMLPMultihead              lact_nvs/lact_ttt.py:150-258

The projections are torch.nn.Linear (hipBLASLt).  Everything between them runs in liblact_hip.so: one kernel turns
the to_qkv output into the operation's q, k, v (silu, per-head L2 norm, head layout), one makes the learning rates
and the momentum, the operation itself, and one kernel turns its output into the o_proj input (per-head RMSNorm,
per-head gate, head layout) -- each with a hand-written backward.  The sliding-window attention of the causal
layer (flash_attn_func in the reference) is torch's scaled_dot_product_attention over blocks of the window size,
which bounds the mask to [window, 2*window] per block.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib
from ._lib import LACT_BF16, LACT_F32
from .minimal import bidirectional_lact_swiglu, block_causal_lact_swiglu, inv_softplus
from .nvs import fast_weight_swish_glu_weight_norm_mini_batch_apply


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _act(t: torch.Tensor):
    if not t.is_cuda:
        raise RuntimeError("lact_amd runs on an MI355X only: tensors must be on a HIP device (no CPU path)")
    if t.dtype == torch.bfloat16:
        return LACT_BF16
    if t.dtype == torch.float32:
        return LACT_F32
    raise TypeError(f"unsupported activation dtype {t.dtype}: bf16 or fp32")


class _PreFn(torch.autograd.Function):
    """qkv [B, L, 3*H*hd] -> q, k, v [(B H), L, hd]."""

    @staticmethod
    def forward(ctx, qkv, H, hd, l2norm):
        qkv = qkv.contiguous()
        B, L, _ = qkv.shape
        q, k, v = (torch.empty((B * H, L, hd), dtype=qkv.dtype, device=qkv.device) for _ in range(3))
        with torch.cuda.device(qkv.device):
            _lib.check(_lib.lib().lact_layer_pre_forward(_act(qkv), B, L, H, hd, int(l2norm), _ptr(qkv), _ptr(q), _ptr(k),
                                                         _ptr(v), _stream(qkv)))
        ctx.save_for_backward(qkv)
        ctx.dims = (B, L, H, hd, int(l2norm))
        return q, k, v

    @staticmethod
    def backward(ctx, dq, dk, dv):
        (qkv,) = ctx.saved_tensors
        B, L, H, hd, l2norm = ctx.dims
        zeros = lambda: torch.zeros((B * H, L, hd), dtype=qkv.dtype, device=qkv.device)
        dq, dk, dv = (zeros() if g is None else g.to(qkv.dtype).contiguous() for g in (dq, dk, dv))
        dqkv = torch.empty_like(qkv)
        with torch.cuda.device(qkv.device):
            _lib.check(_lib.lib().lact_layer_pre_backward(_act(qkv), B, L, H, hd, l2norm, _ptr(qkv), _ptr(dq), _ptr(dk),
                                                          _ptr(dv), _ptr(dqkv), _stream(qkv)))
        return dqkv, None, None, None


class _LrFn(torch.autograd.Function):
    """lr_raw [B, L, 3*H] (head-major with three rates per head, or rate-major when rates_major), momentum_raw
    [B, L, H] or None -> lr0, lr1, lr2, momentum [(B H), L, 1] fp32."""

    @staticmethod
    def forward(ctx, lr_raw, mom_raw, H, base_lr_inv, rates_major=False):
        lr_raw = lr_raw.float().contiguous()
        mom_c = None if mom_raw is None else mom_raw.float().contiguous()
        B, L, _ = lr_raw.shape
        outs = [torch.empty((B * H, L, 1), dtype=torch.float32, device=lr_raw.device) for _ in range(3)]
        mom = torch.empty((B * H, L, 1), dtype=torch.float32, device=lr_raw.device) if mom_c is not None else None
        with torch.cuda.device(lr_raw.device):
            _lib.check(_lib.lib().lact_layer_lr_forward(B, L, H, int(rates_major), float(base_lr_inv), _ptr(lr_raw), _ptr(outs[0]),
                                                        _ptr(outs[1]), _ptr(outs[2]), _ptr(mom_c), _ptr(mom),
                                                        _stream(lr_raw)))
        ctx.save_for_backward(lr_raw, mom_c)
        ctx.dims = (B, L, H, float(base_lr_inv), int(rates_major))
        ctx.mom_dtype = None if mom_raw is None else mom_raw.dtype
        if mom is None:
            return outs[0], outs[1], outs[2]
        return outs[0], outs[1], outs[2], mom

    @staticmethod
    def backward(ctx, d0, d1, d2, dm=None):
        lr_raw, mom_c = ctx.saved_tensors
        B, L, H, base, rates_major = ctx.dims
        c = lambda g: None if g is None else g.float().contiguous()
        d0, d1, d2, dm = c(d0), c(d1), c(d2), c(dm)
        dlr_raw = torch.empty_like(lr_raw)
        dmom_raw = torch.empty_like(mom_c) if mom_c is not None else None
        with torch.cuda.device(lr_raw.device):
            _lib.check(_lib.lib().lact_layer_lr_backward(B, L, H, rates_major, base, _ptr(lr_raw), _ptr(d0), _ptr(d1), _ptr(d2),
                                                         _ptr(dlr_raw), _ptr(mom_c), _ptr(dm), _ptr(dmom_raw),
                                                         _stream(lr_raw)))
        return dlr_raw, (None if dmom_raw is None else dmom_raw.to(ctx.mom_dtype)), None, None, None


class _PostFn(torch.autograd.Function):
    """o [(B H), L, hd] -> y [B, L, H*hd]: RMSNorm(weight) per head if weight is given or use_norm, times
    silu(gate_raw [B, L, H]) if given."""

    @staticmethod
    def forward(ctx, o, weight, gate_raw, B, H, use_norm, eps):
        o = o.contiguous()
        _, L, hd = o.shape
        w = None if weight is None else weight.float().contiguous()
        g = None if gate_raw is None else gate_raw.to(o.dtype).contiguous()
        y = torch.empty((B, L, H * hd), dtype=o.dtype, device=o.device)
        with torch.cuda.device(o.device):
            _lib.check(_lib.lib().lact_layer_post_forward(_act(o), B, L, H, hd, int(use_norm), float(eps), _ptr(o), _ptr(w),
                                                          _ptr(g), _ptr(y), _stream(o)))
        ctx.save_for_backward(o, w, g)
        ctx.dims = (B, L, H, hd, int(use_norm), float(eps))
        ctx.dtypes = (None if weight is None else weight.dtype, None if gate_raw is None else gate_raw.dtype)
        return y

    @staticmethod
    def backward(ctx, dy):
        o, w, g = ctx.saved_tensors
        B, L, H, hd, use_norm, eps = ctx.dims
        lib = _lib.lib()
        dy = dy.to(o.dtype).contiguous()
        d_o = torch.empty_like(o)
        dg = torch.empty_like(g) if g is not None else None
        rows = lib.lact_layer_post_dw_rows(B, L, H)
        dw_part = torch.empty((rows, hd), dtype=torch.float32, device=o.device) if (use_norm and w is not None) else None
        with torch.cuda.device(o.device):
            _lib.check(lib.lact_layer_post_backward(_act(o), B, L, H, hd, use_norm, eps, _ptr(o), _ptr(w), _ptr(g), _ptr(dy),
                                                    _ptr(d_o), _ptr(dg), _ptr(dw_part), _stream(o)))
        wd, gd = ctx.dtypes
        dw = None if dw_part is None else dw_part.sum(dim=0).to(wd)
        return d_o, dw, (None if dg is None else dg.to(gd)), None, None, None, None


def _fast_weights(layer, B):
    """[nh, ...] parameters -> [(B nh), ...] (bidirectional_lact_layer.py:259-261)."""
    return tuple(w.repeat(B, 1, 1) for w in (layer.w0, layer.w1, layer.w2))


def _norm_args(o_norm):
    if isinstance(o_norm, nn.RMSNorm):
        return o_norm.weight, True, (o_norm.eps if o_norm.eps is not None else 1e-5)
    return None, False, 1e-5


class BidirectionalLaCTSwiGLU(nn.Module):
    """bidirectional_lact_layer.py:171-270."""

    def __init__(self, dim: int, head_dim: int, inter_multi: float = 1, use_o_norm: bool = True,
                 qk_l2_norm: bool = True, use_muon: bool = True, base_lr: float = 1e-2):
        super().__init__()
        self.dim, self.head_dim, self.inter_multi = dim, head_dim, inter_multi
        self.use_o_norm, self.qk_l2_norm, self.use_muon = use_o_norm, qk_l2_norm, use_muon
        self.num_heads = dim // head_dim
        self.to_qkv = nn.Linear(dim, 3 * dim, bias=False)
        self.o_proj = nn.Linear(dim, dim, bias=False)
        self.lr_dim = 1
        self.lr_proj = nn.Linear(dim, self.lr_dim * 3 * self.num_heads, bias=False)
        self.base_lr = base_lr
        self.base_lr_inv = inv_softplus(base_lr)
        d_in, d_out, d_h = head_dim, head_dim, int(head_dim * inter_multi)
        self.w0 = nn.Parameter(torch.randn(self.num_heads, d_h, d_in) / math.sqrt(d_in))
        self.w1 = nn.Parameter(torch.randn(self.num_heads, d_out, d_h) / math.sqrt(d_h))
        self.w2 = nn.Parameter(torch.randn(self.num_heads, d_h, d_in) / math.sqrt(d_in))
        self.o_norm = nn.RMSNorm(head_dim, eps=1e-5, elementwise_affine=True) if use_o_norm else nn.Identity()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x: [b, l, d] -> [b, l, d]"""
        B = x.shape[0]
        q, k, v = _PreFn.apply(self.to_qkv(x), self.num_heads, self.head_dim, self.qk_l2_norm)
        with torch.autocast(device_type="cuda", enabled=False):      # the reference keeps the rates out of autocast (:247-249)
            lr_raw = self.lr_proj(x)
        lr0, lr1, lr2 = _LrFn.apply(lr_raw, None, self.num_heads, self.base_lr_inv)
        w0, w1, w2 = _fast_weights(self, B)
        o = bidirectional_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, self.use_muon)
        weight, use_norm, eps = _norm_args(self.o_norm)
        return self.o_proj(_PostFn.apply(o, weight, None, B, self.num_heads, use_norm, eps))


def sliding_window_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: Optional[int]) -> torch.Tensor:
    """q, k, v: [b, l, h, d].  Causal attention where query i sees keys i-(window-1) .. i -- what the reference asks
    of flash_attn_func(causal=True, window_size=(window-1, 0)) (causal_lact_with_sliding_window_attn.py:371-375).
    Query blocks of `window` rows attend to their own and the previous block under a band mask."""
    b, l, h, d = q.shape
    q, k, v = (t.transpose(1, 2) for t in (q, k, v))              # [b, h, l, d]
    if window is None or window >= l:
        return F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2)
    outs = []
    for s in range(0, l, window):
        e = min(s + window, l)
        ks = max(0, s - window + 1)
        qi = torch.arange(s, e, device=q.device)[:, None]
        kj = torch.arange(ks, e, device=q.device)[None, :]
        mask = (kj <= qi) & (kj >= qi - (window - 1))
        outs.append(F.scaled_dot_product_attention(q[:, :, s:e], k[:, :, ks:e], v[:, :, ks:e], attn_mask=mask))
    return torch.cat(outs, dim=2).transpose(1, 2)


class CausalLaCTSwiGLUWithSlidingWindowAttn(nn.Module):
    """causal_lact_with_sliding_window_attn.py:222-391."""

    def __init__(self, dim: int, head_dim: int, attn_head_dim: int, lact_chunk_size: int = 2048, window_size: int = 2048,
                 inter_multi: float = 1, use_o_norm: bool = True, use_momentum: bool = True, use_muon: bool = True,
                 base_lr: float = 1e-2, ttt_scale_before_sum: bool = True):
        super().__init__()
        self.dim, self.head_dim, self.attn_head_dim, self.inter_multi = dim, head_dim, attn_head_dim, inter_multi
        self.lact_chunk_size, self.window_size, self.use_o_norm = lact_chunk_size, window_size, use_o_norm
        self.num_ttt_heads, self.num_attn_heads = dim // head_dim, dim // attn_head_dim
        self.to_qkv = nn.Linear(dim, 3 * dim, bias=False)
        self.o_proj = nn.Linear(dim, dim, bias=False)
        self.lr_dim = 1
        self.lr_proj = nn.Linear(dim, self.lr_dim * 3 * self.num_ttt_heads, bias=False)
        self.base_lr = base_lr
        self.base_lr_inv = inv_softplus(base_lr)
        d_in, d_out, d_h = head_dim, head_dim, int(head_dim * inter_multi)
        self.w0 = nn.Parameter(torch.randn(self.num_ttt_heads, d_h, d_in) / math.sqrt(d_in))
        self.w1 = nn.Parameter(torch.randn(self.num_ttt_heads, d_out, d_h) / math.sqrt(d_h))
        self.w2 = nn.Parameter(torch.randn(self.num_ttt_heads, d_h, d_in) / math.sqrt(d_in))
        self.use_muon, self.use_momentum = use_muon, use_momentum
        if use_momentum:
            self.momentum_proj = nn.Sequential(nn.Linear(dim, self.num_ttt_heads), nn.Sigmoid())
        self.o_norm = nn.RMSNorm(head_dim, eps=1e-5, elementwise_affine=True) if use_o_norm else nn.Identity()
        self.qk_scale = nn.Parameter(torch.ones(dim, 2))
        self.qk_offset = nn.Parameter(torch.zeros(dim, 2))
        # the reference creates this only when ttt_scale_before_sum, and its forward always uses it (:348)
        self.ttt_scale_proj = nn.Linear(dim, self.num_ttt_heads)

    def _rescale_qk(self, q, k):
        dt = q.dtype
        q = q * self.qk_scale[:, 0] + self.qk_offset[:, 0]
        k = k * self.qk_scale[:, 1] + self.qk_offset[:, 1]
        return q.to(dt), k.to(dt)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x: [b, l, d] -> [b, l, d]"""
        B, L, _ = x.shape
        H = self.num_ttt_heads
        attn_qkv = self.to_qkv(x)
        q, k, v = _PreFn.apply(attn_qkv, H, self.head_dim, True)
        with torch.autocast(device_type="cuda", enabled=False):
            lr_raw = self.lr_proj(x)
        mom_raw = self.momentum_proj[0](x) if self.use_momentum else None      # the Sigmoid of the Sequential is in the kernel
        res = _LrFn.apply(lr_raw, mom_raw, H, self.base_lr_inv)
        lr0, lr1, lr2 = res[:3]
        momentum = res[3] if self.use_momentum else None
        w0, w1, w2 = _fast_weights(self, B)
        o = block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum, self.use_muon,
                                     chunk_size=self.lact_chunk_size)
        weight, use_norm, eps = _norm_args(self.o_norm)
        ttt = _PostFn.apply(o, weight, self.ttt_scale_proj(x), B, H, use_norm, eps)
        aq, ak, av = attn_qkv.chunk(3, dim=-1)
        aq, ak = self._rescale_qk(aq, ak)
        sh = lambda t: t.reshape(B, L, self.num_attn_heads, self.attn_head_dim)
        attn = sliding_window_attention(sh(aq), sh(ak), sh(av), self.window_size).reshape(B, L, -1)
        return self.o_proj(attn + ttt)


class FastWeightGluMLPMultihead(nn.Module):
    """lact_nvs/lact_ttt.py:150-258: the layer of the novel-view-synthesis model.  Fast weights in the transposed
    layout (w0, w2: [nh, d, dh]; w1: [nh, dh, d]); `info["ttt_op_order"]` is the list of TTTOperator steps and
    `info["w0"/"w1"/"w2"]`, when present, are the fast weights a previous call returned (state carried from the
    reconstruction pass into the rendering pass, lact_nvs/model.py:272-384)."""

    def __init__(self, dim: int, head_dim: int, inter_multi: int = 1, bias: bool = False, base_lr: float = 0.01,
                 muon_update_steps: int = 0):
        super().__init__()
        assert dim % head_dim == 0
        self.dim, self.num_heads, self.muon_update_steps = dim, dim // head_dim, muon_update_steps
        self.head_dim = head_dim
        d_in = d_out = head_dim
        d_h = int(head_dim * inter_multi)
        gain = math.sqrt(2)
        self.w0 = nn.Parameter(torch.randn(self.num_heads, d_in, d_h) * gain / math.sqrt(d_in))
        self.w1 = nn.Parameter(torch.randn(self.num_heads, d_h, d_out) * gain / math.sqrt(d_h))
        self.w2 = nn.Parameter(torch.randn(self.num_heads, d_in, d_h) * gain / math.sqrt(d_in))
        self.to_qkv = nn.Linear(dim, 3 * dim, bias=bias)
        self.c_proj = nn.Linear(dim, dim, bias=bias)
        self.lr_dim = self.num_heads
        self.lr_fc = nn.Linear(dim, self.lr_dim * 3)
        self.base_lr_inv = inv_softplus(base_lr)
        self.o_norm = nn.RMSNorm(head_dim, eps=1e-5, elementwise_affine=True)

    def forward(self, x: torch.Tensor, info={}, *args):
        """x: [b, l, d] -> ([b, l', d], {"w0", "w1", "w2"}) with l' the rows of the apply steps in program order."""
        B = x.shape[0]
        q, k, v = _PreFn.apply(self.to_qkv(x), self.num_heads, self.head_dim, True)          # :203-210
        with torch.autocast(device_type="cuda", enabled=False):                              # :212-213
            lr_raw = self.lr_fc(x.float())
        lr0, lr1, lr2 = _LrFn.apply(lr_raw, None, self.num_heads, self.base_lr_inv, True)    # '(lrs h d)', :215-219
        if "w0" in info:                                                                      # :221-229
            assert "w1" in info and "w2" in info
            w0, w1, w2 = info["w0"], info["w1"], info["w2"]
        else:
            w0, w1, w2 = _fast_weights(self, B)
        o, w0, w1, w2 = fast_weight_swish_glu_weight_norm_mini_batch_apply(
            w0, w1, w2, q, k, v, lr0, lr1, lr2, info["ttt_op_order"], muon_update_steps=self.muon_update_steps)
        weight, use_norm, eps = _norm_args(self.o_norm)
        y = _PostFn.apply(o, weight, None, B, self.num_heads, use_norm, eps)
        return self.c_proj(y), {"w0": w0, "w1": w1, "w2": w2}
