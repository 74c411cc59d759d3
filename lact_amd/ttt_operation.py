"""Drop-in for lact_llm/lact_model/ttt_operation.py: same function names, argument order and
defaults; the arithmetic runs in liblact_hip.so."""
from __future__ import annotations

from typing import Optional

import torch

from . import ops
from .ops import NS5_COEFFS, Program, block_causal_steps, run_program


def silu_backprop(dy: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """ttt_operation.py:5-17 (layer-side helper; inside the operation this is fused into the GEMM epilogues)."""
    sigma = torch.sigmoid(x)
    return dy * sigma * (1 + x * (1 - sigma))


def l2_norm(x: torch.Tensor) -> torch.Tensor:
    """ttt_operation.py:20-27 (layer-side pre-processing of q and k)."""
    return (x / (x.float().norm(dim=-1, keepdim=True) + 1e-5)).type(x.dtype)


def zeropower_via_newtonschulz5(G: torch.Tensor) -> torch.Tensor:
    """ttt_operation.py:30-66."""
    return ops.newton_schulz(G, NS5_COEFFS, ns_mode=ops.NS_AUTOCAST if torch.is_autocast_enabled() else ops.NS_PLAIN_BF16)


def _block_causal(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon, momentum, prenorm,
                  muon_stacked=False, renorm_eps_in_sqrt=False):
    prog = Program(steps=block_causal_steps(k.shape[1], chunk_size), out_len=q.shape[1], return_state=False,
                   ns_coeffs=NS5_COEFFS if use_muon else None, prenorm=prenorm,
                   ns_mode=ops._ns_mode(q), muon_stacked=muon_stacked and use_muon,
                   renorm_eps_in_sqrt=renorm_eps_in_sqrt)
    out, _, _ = run_program(prog, w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum)
    return out


def block_causal_lact_swiglu(w0: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, q: torch.Tensor, k: torch.Tensor,
                             v: torch.Tensor, lr0: torch.Tensor, lr1: torch.Tensor, lr2: torch.Tensor,
                             chunk_size: int = 2048, use_muon: bool = False,
                             momentum: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ttt_operation.py:71-214.  w0,w2 [b,dh,dk], w1 [b,dv,dh], q,k,v [b,l,d], lr*, momentum [b,l,1] -> [b,l,dv]."""
    return _block_causal(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon, momentum, False)


def prenorm_block_causal_lact_swiglu(w0: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, q: torch.Tensor,
                                     k: torch.Tensor, v: torch.Tensor, lr0: torch.Tensor, lr1: torch.Tensor,
                                     lr2: torch.Tensor, chunk_size: int = 2048, use_muon: bool = False,
                                     momentum: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ttt_operation.py:219-364."""
    return _block_causal(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon, momentum, True)


def postnorm_block_causal_lact_swiglu_fused_kernel_triton(w0: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                                                          q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                                          lr0: torch.Tensor, lr1: torch.Tensor, lr2: torch.Tensor,
                                                          chunk_size: int = 2048, use_muon: bool = False,
                                                          momentum: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ttt_operation_fused_kernel.py:67-199 (the layer's `use_fused_kernel=True` path, layer_lact_swiglu.py:525-528):
    same schedule as block_causal_lact_swiglu; Muon orthogonalises cat(dw0, dw2) as one [2dh, d] matrix and the
    row renorm has eps inside the sqrt."""
    return _block_causal(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon, momentum, False,
                         muon_stacked=True, renorm_eps_in_sqrt=True)


def prenorm_block_causal_lact_swiglu_fused_kernel_triton(w0: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                                                         q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                                         lr0: torch.Tensor, lr1: torch.Tensor, lr2: torch.Tensor,
                                                         chunk_size: int = 2048, use_muon: bool = False,
                                                         momentum: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ttt_operation_fused_kernel.py:202-338 (layer_lact_swiglu.py:493-496): pre-norm accumulator, stacked Muon,
    eps outside the sqrt (:322-327)."""
    return _block_causal(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon, momentum, True, muon_stacked=True)
