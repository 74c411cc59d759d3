"""Drop-ins for the operations of minimal_implementations/ (argument orders of that directory)."""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import ops
from ._lib import LACT_APPLY, LACT_UPDATE
from .ops import NS5_COEFFS, Program, run_program
from .ttt_operation import _block_causal, l2_norm, silu_backprop, zeropower_via_newtonschulz5  # noqa: F401


def inv_softplus(x):
    """bidirectional_lact_layer.py:163-168."""
    if isinstance(x, torch.Tensor):
        return x + torch.log(-torch.expm1(-x))
    return x + math.log(-math.expm1(-x))


def block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, momentum: Optional[torch.Tensor] = None,
                             use_muon: bool = True, chunk_size: int = 2048) -> torch.Tensor:
    """causal_lact_with_sliding_window_attn.py:84-211 (momentum, use_muon, chunk_size order of :94-96)."""
    return _block_causal(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size, use_muon, momentum, False)


def bidirectional_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, use_muon: bool = True,
                              muon_mode: str = "reference") -> torch.Tensor:
    """bidirectional_lact_layer.py:74-160: one update on every token, then apply to every query.
    muon_mode="reference" reproduces :139-146 (the orthogonalised gradient replaces the weight and the
    raw gradient is added); "intended" adds the orthogonalised gradient to the weight."""
    prog = Program(steps=((LACT_UPDATE, 0, k.shape[1], 0), (LACT_APPLY, 0, q.shape[1], 0)), out_len=q.shape[1], return_state=False,
                   ns_coeffs=NS5_COEFFS if use_muon else None,
                   muon_replaces_weight=(use_muon and muon_mode == "reference"),
                   ns_mode=ops._ns_mode(q))
    out, _, _ = run_program(prog, w0, w1, w2, q, k, v, lr0, lr1, lr2, None)
    return out
