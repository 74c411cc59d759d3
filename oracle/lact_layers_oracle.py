"""CPU restatement of the reference's layer classes around the TTT operation.  TEST INFRASTRUCTURE ONLY:
nothing in the product imports this module; tests compare the HIP-backed layers in lact_amd/layers.py with it.

  BidirectionalLaCTSwiGLU                minimal_implementations/bidirectional_lact_layer.py:171-270
  CausalLaCTSwiGLUWithSlidingWindowAttn  minimal_implementations/causal_lact_with_sliding_window_attn.py:222-391
  FastWeightGluMLPMultihead              lact_nvs/lact_ttt.py:150-258

Parameter names equal the reference's, so a state_dict moves between the three implementations.  The operation
inside is the oracle's (oracle/lact_oracle.py).  The sliding-window attention of the causal layer, which the
reference computes with flash_attn_func(causal=True, window_size=(W-1, 0)), is written as an explicit masked
softmax: query i sees keys j with i-(W-1) <= j <= i, scale 1/sqrt(attn_head_dim).

Pinned by tests/golden/bidirectional_layer_cpu_fp32.npz (the reference's own bidirectional layer run on the CPU:
output and every gradient); the causal layer shares all of that code path except momentum head, per-head gate,
q/k rescale and the attention branch, which are pinned by closed-form checks in tests/test_oracle_layers.py.
The novel-view-synthesis layer (rate-major learning-rate layout, transposed fast weights, weights carried through
`info`) is pinned there too: against a per-head composition written with explicit loops, and by the identity
"update in one call, apply in the next with the returned weights" == "update and apply in one call".
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import lact_oracle as O


def _heads(t: torch.Tensor, n: int, h: int, d: int):
    """'b l (n h d) -> n (b h) l d'"""
    b, l, _ = t.shape
    return t.reshape(b, l, n, h, d).permute(2, 0, 3, 1, 4).reshape(n, b * h, l, d)


def _unheads(t: torch.Tensor, b: int, h: int):
    """'(b h) l d -> b l (h d)'"""
    bh, l, d = t.shape
    return t.reshape(b, h, l, d).permute(0, 2, 1, 3).reshape(b, l, h * d)


class BidirectionalLaCTSwiGLU(nn.Module):
    """bidirectional_lact_layer.py:171-270."""

    def __init__(self, dim: int, head_dim: int, inter_multi: float = 1, use_o_norm: bool = True,
                 qk_l2_norm: bool = True, use_muon: bool = True, base_lr: float = 1e-2,
                 num: O.Numerics = O.Numerics()):
        super().__init__()
        self.dim, self.head_dim, self.num_heads = dim, head_dim, dim // head_dim
        self.to_qkv = nn.Linear(dim, 3 * dim, bias=False)
        self.o_proj = nn.Linear(dim, dim, bias=False)
        self.lr_proj = nn.Linear(dim, 3 * self.num_heads, bias=False)
        self.base_lr_inv = O.inv_softplus(base_lr)
        d_h = int(head_dim * inter_multi)
        self.w0 = nn.Parameter(torch.randn(self.num_heads, d_h, head_dim) / math.sqrt(head_dim))
        self.w1 = nn.Parameter(torch.randn(self.num_heads, head_dim, d_h) / math.sqrt(d_h))
        self.w2 = nn.Parameter(torch.randn(self.num_heads, d_h, head_dim) / math.sqrt(head_dim))
        self.qk_l2_norm, self.use_muon = qk_l2_norm, use_muon
        self.o_norm = nn.RMSNorm(head_dim, eps=1e-5, elementwise_affine=True) if use_o_norm else nn.Identity()
        self.num = num

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        B = x.shape[0]
        qkv = F.silu(self.to_qkv(x))                                                   # :231
        q, k, v = _heads(qkv, 3, self.num_heads, self.head_dim)                        # :234-240
        if self.qk_l2_norm:                                                            # :242-244
            q, k = O.l2_norm(q, self.num), O.l2_norm(k, self.num)
        lr = F.softplus(self.lr_proj(x).float() + self.base_lr_inv)                    # :248-251
        lr0, lr1, lr2 = _heads(lr.reshape(B, x.shape[1], self.num_heads, 3).permute(0, 1, 3, 2).reshape(B, x.shape[1], -1),
                               3, self.num_heads, 1)                                   # 'b l (h lrs d) -> lrs (b h) l d', :254-256
        w0, w1, w2 = (w.repeat(B, 1, 1) for w in (self.w0, self.w1, self.w2))          # :259-261
        o = O.bidirectional_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, self.use_muon, num=self.num)   # :264-266
        o = self.o_norm(o)
        return self.o_proj(_unheads(o, B, self.num_heads))                             # :268-272


def sliding_window_attention(q, k, v, window):
    """q, k, v: [b, l, h, d].  Causal attention where query i sees keys i-(window-1) .. i
    (flash_attn_func(causal=True, window_size=(window-1, 0)); window None = plain causal)."""
    b, l, h, d = q.shape
    ct = torch.promote_types(q.dtype, torch.float32)
    s = torch.einsum("bihd,bjhd->bhij", q.to(ct), k.to(ct)) / math.sqrt(d)
    i = torch.arange(l)[:, None]
    j = torch.arange(l)[None, :]
    mask = j <= i
    if window is not None:
        mask = mask & (j >= i - (window - 1))
    s = s.masked_fill(~mask, float("-inf"))
    return torch.einsum("bhij,bjhd->bihd", torch.softmax(s, dim=-1), v.to(ct)).to(q.dtype)


class CausalLaCTSwiGLUWithSlidingWindowAttn(nn.Module):
    """causal_lact_with_sliding_window_attn.py:222-391."""

    def __init__(self, dim: int, head_dim: int, attn_head_dim: int, lact_chunk_size: int = 2048, window_size: int = 2048,
                 inter_multi: float = 1, use_o_norm: bool = True, use_momentum: bool = True, use_muon: bool = True,
                 base_lr: float = 1e-2, ttt_scale_before_sum: bool = True, num: O.Numerics = O.Numerics()):
        super().__init__()
        self.dim, self.head_dim, self.attn_head_dim = dim, head_dim, attn_head_dim
        self.lact_chunk_size, self.window_size = lact_chunk_size, window_size
        self.num_ttt_heads, self.num_attn_heads = dim // head_dim, dim // attn_head_dim
        self.to_qkv = nn.Linear(dim, 3 * dim, bias=False)
        self.o_proj = nn.Linear(dim, dim, bias=False)
        self.lr_proj = nn.Linear(dim, 3 * self.num_ttt_heads, bias=False)
        self.base_lr_inv = O.inv_softplus(base_lr)
        d_h = int(head_dim * inter_multi)
        self.w0 = nn.Parameter(torch.randn(self.num_ttt_heads, d_h, head_dim) / math.sqrt(head_dim))
        self.w1 = nn.Parameter(torch.randn(self.num_ttt_heads, head_dim, d_h) / math.sqrt(d_h))
        self.w2 = nn.Parameter(torch.randn(self.num_ttt_heads, d_h, head_dim) / math.sqrt(head_dim))
        self.use_muon, self.use_momentum = use_muon, use_momentum
        if use_momentum:
            self.momentum_proj = nn.Sequential(nn.Linear(dim, self.num_ttt_heads), nn.Sigmoid())
        self.o_norm = nn.RMSNorm(head_dim, eps=1e-5, elementwise_affine=True) if use_o_norm else nn.Identity()
        self.qk_scale = nn.Parameter(torch.ones(dim, 2))
        self.qk_offset = nn.Parameter(torch.zeros(dim, 2))
        self.ttt_scale_proj = nn.Linear(dim, self.num_ttt_heads)     # the reference's forward needs it (:348)
        self.num = num

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        B, L, _ = x.shape
        H = self.num_ttt_heads
        attn_qkv = self.to_qkv(x)                                                      # :312
        q, k, v = _heads(F.silu(attn_qkv), 3, H, self.head_dim)                        # :313-321
        q, k = O.l2_norm(q, self.num), O.l2_norm(k, self.num)                          # :322
        lr = F.softplus(self.lr_proj(x).float() + self.base_lr_inv)                    # :326-329
        lr0, lr1, lr2 = _heads(lr.reshape(B, L, H, 3).permute(0, 1, 3, 2).reshape(B, L, -1), 3, H, 1)   # :332-334
        w0, w1, w2 = (w.repeat(B, 1, 1) for w in (self.w0, self.w1, self.w2))
        momentum = None
        if self.use_momentum:                                                          # :341-345
            momentum = _heads(self.momentum_proj(x), 1, H, 1)[0]
        o = O.block_causal_lact_swiglu_minimal(w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum, self.use_muon,
                                               chunk_size=self.lact_chunk_size, num=self.num)           # :348-350
        o = self.o_norm(o)                                                             # :351
        gate = _heads(F.silu(self.ttt_scale_proj(x)), 1, H, 1)[0]                      # :352-353
        ttt = _unheads(o * gate, B, H)                                                 # :354-357
        aq, ak, av = attn_qkv.chunk(3, dim=-1)                                         # :361
        dt = aq.dtype                                                                  # _rescale_qk, :295-309
        aq = (aq * self.qk_scale[:, 0] + self.qk_offset[:, 0]).to(dt)
        ak = (ak * self.qk_scale[:, 1] + self.qk_offset[:, 1]).to(dt)
        sh = lambda t: t.reshape(B, L, self.num_attn_heads, self.attn_head_dim)
        attn = sliding_window_attention(sh(aq), sh(ak), sh(av), self.window_size).reshape(B, L, -1)   # :371-377
        return self.o_proj(attn + ttt)                                                 # :379-382


class FastWeightGluMLPMultihead(nn.Module):
    """lact_nvs/lact_ttt.py:150-258."""

    def __init__(self, dim: int, head_dim: int, inter_multi: int = 1, bias: bool = False, base_lr: float = 0.01,
                 muon_update_steps: int = 0, num: O.Numerics = O.Numerics()):
        super().__init__()
        self.dim, self.head_dim, self.num_heads = dim, head_dim, dim // head_dim
        self.muon_update_steps = muon_update_steps
        d_h = int(head_dim * inter_multi)
        gain = math.sqrt(2)
        self.w0 = nn.Parameter(torch.randn(self.num_heads, head_dim, d_h) * gain / math.sqrt(head_dim))   # :186-194
        self.w1 = nn.Parameter(torch.randn(self.num_heads, d_h, head_dim) * gain / math.sqrt(d_h))
        self.w2 = nn.Parameter(torch.randn(self.num_heads, head_dim, d_h) * gain / math.sqrt(head_dim))
        self.to_qkv = nn.Linear(dim, 3 * dim, bias=bias)
        self.c_proj = nn.Linear(dim, dim, bias=bias)
        self.lr_fc = nn.Linear(dim, self.num_heads * 3)
        self.base_lr_inv = O.inv_softplus(base_lr)
        self.o_norm = nn.RMSNorm(head_dim, eps=1e-5, elementwise_affine=True)
        self.num = num

    def forward(self, x: torch.Tensor, info={}, *args):
        B, L, _ = x.shape
        H = self.num_heads
        qkv = F.silu(self.to_qkv(x))                                                   # :203
        q, k, v = _heads(qkv, 3, H, self.head_dim)                                     # :204-207
        q, k = O.l2_norm(q, self.num), O.l2_norm(k, self.num)                          # :208-209
        lr = F.softplus(self.lr_fc(x.to(torch.promote_types(x.dtype, torch.float32))) + self.base_lr_inv)   # :211-214
        lr0, lr1, lr2 = _heads(lr, 3, H, 1)                                            # 'b l (lrs h d) -> lrs (b h) l d', :215-218
        if "w0" in info:                                                               # :220-228
            w0, w1, w2 = info["w0"], info["w1"], info["w2"]
        else:
            w0, w1, w2 = (w.repeat(B, 1, 1) for w in (self.w0, self.w1, self.w2))
        o, w0, w1, w2 = O.fast_weight_swish_glu_weight_norm_mini_batch_apply(
            w0, w1, w2, q, k, v, lr0, lr1, lr2, info["ttt_op_order"], muon_update_steps=self.muon_update_steps,
            num=self.num)                                                              # :230-233
        o = self.o_norm(o)                                                             # :235
        return self.c_proj(_unheads(o, B, H)), {"w0": w0, "w1": w1, "w2": w2}          # :236-241
