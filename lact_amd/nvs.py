"""Drop-in for the operation of lact_nvs/lact_ttt.py (transposed weight layout, update/apply program)."""
from __future__ import annotations

import collections

import torch

from . import ops
from ._lib import LACT_APPLY, LACT_UPDATE
from .ops import NS_CLASSIC, Program, run_program

TTTOperator = collections.namedtuple("TTTOperator", ["start", "end", "update", "apply"])  # lact_ttt.py:10


def zeropower_via_newtonschulz5(G: torch.Tensor, steps: int) -> torch.Tensor:
    """lact_ttt.py:33-67."""
    return ops.newton_schulz(G, (NS_CLASSIC,) * steps, ns_mode=ops.NS_AUTOCAST if torch.is_autocast_enabled() else ops.NS_PLAIN_BF16)


def fast_weight_swish_glu_weight_norm_mini_batch_apply(w0, w1, w2, q, k, v, lr0, lr1, lr2, ttt_ua_order,
                                                       muon_update_steps: int = 0):
    """lact_ttt.py:71-147.  w0, w2: [b, d, dh]; w1: [b, dh, d]; returns (output, w0, w1, w2).
    Outputs of the apply operators are concatenated in program order (:142-145); the initial row norms
    are detached (:96-98); Newton-Schulz always runs, with `muon_update_steps` iterations (:120-128)."""
    steps, pos = [], 0
    for start, end, update, apply in ttt_ua_order:
        if update:
            steps.append((LACT_UPDATE, start, end, 0))
        if apply:
            steps.append((LACT_APPLY, start, end, pos))
            pos += end - start
    prog = Program(steps=tuple(steps), out_len=pos, ns_coeffs=(NS_CLASSIC,) * muon_update_steps,
                   detach_norms=True, ns_mode=ops._ns_mode(q))
    out, (a0, a1, a2), _ = run_program(prog, w0.transpose(1, 2), w1.transpose(1, 2), w2.transpose(1, 2),
                                       q, k, v, lr0, lr1, lr2, None)
    return out, a0.transpose(1, 2), a1.transpose(1, 2), a2.transpose(1, 2)
