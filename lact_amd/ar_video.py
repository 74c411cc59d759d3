"""Drop-ins for the operations of lact_ar_video/minVid/models/blocks/ar_lact_swa_repeat{,_sp}.py."""
from __future__ import annotations

from typing import Optional

import torch

from . import ops
from ._lib import LACT_APPLY, LACT_UPDATE
from .ops import NS_CLASSIC, Program, run_program


def zeropower_via_newtonschulz5(G: torch.Tensor, steps: int) -> torch.Tensor:
    """functions.py:38-72."""
    return ops.newton_schulz(G, (NS_CLASSIC,) * steps, ns_mode=ops.NS_AUTOCAST if torch.is_autocast_enabled() else ops.NS_PLAIN_BF16)


def _ar_steps(seq_len, q_len, mini_batch_size, update_length, update_every, num_repeat):
    """ar_lact_swa_repeat.py:76-101,104-165."""
    if update_length == -1:
        update_length = seq_len
    if mini_batch_size == -1:
        mini_batch_size = update_length
    if update_every == -1:
        update_every = mini_batch_size * 2
    first = update_every - mini_batch_size
    steps = [(LACT_APPLY, 0, min(first, q_len), 0)]
    for _ in range(num_repeat):
        for s in range(first, update_length, update_every):
            steps.append((LACT_UPDATE, s, min(s + mini_batch_size, seq_len), 0))   # slices stop at the end (:79-82)
            steps.append((LACT_APPLY, s, min(s + update_every, q_len), s))
    return tuple(steps)


def _scaled(lr, w_scale: float):
    """The reference forms (k * lr) * w_scale, left to right (ar_lact_swa_repeat.py:134-138); the kernels take one
    per-token factor, so lr * w_scale is folded first.  The two agree bit for bit when w_scale is a power of two --
    the layer's only value is 1.0 (ar_lact_swa_repeat.py:629) -- and otherwise differ by one fp32 rounding in front of
    the bf16 cast of the GEMM operand."""
    return lr if w_scale == 1.0 else lr * w_scale


def ar_fast_weight_swish_glu_weight_norm_mini_batch_with_momentum(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale: float, num_repeat: int = 1, mini_batch_size: int = -1,
        update_length: int = -1, update_every: int = -1, use_moun: bool = False, num_moun_iters: int = 3,
        weight_norm: bool = True, fw_momentum: Optional[torch.Tensor] = None, use_momentum: bool = False):
    """ar_lact_swa_repeat_sp.py:28-193.  Returns (output, w0, w1, w2)."""
    prog = Program(steps=_ar_steps(k.shape[1], q.shape[1], mini_batch_size, update_length, update_every, num_repeat),
                   out_len=q.shape[1], ns_coeffs=(NS_CLASSIC,) * num_moun_iters if use_moun else None,
                   weight_norm=weight_norm, ns_mode=ops._ns_mode(q))
    out, ws, _ = run_program(prog, w0, w1, w2, q, k, v, _scaled(lr0, w_scale), _scaled(lr1, w_scale), _scaled(lr2, w_scale),
                             fw_momentum if use_momentum else None)
    return (out,) + tuple(ws)


def ar_fast_weight_swish_glu_weight_norm_mini_batch(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale: float, num_repeat: int = 1, mini_batch_size: int = -1,
        update_length: int = -1, update_every: int = -1, use_moun: bool = False, num_moun_iters: int = 3,
        weight_norm: bool = True):
    """ar_lact_swa_repeat.py:23-168."""
    return ar_fast_weight_swish_glu_weight_norm_mini_batch_with_momentum(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale, num_repeat, mini_batch_size, update_length, update_every,
        use_moun, num_moun_iters, weight_norm)


def ar_fast_weight_swish_glu_weight_norm_mini_batch_inference(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale: float, num_repeat: int = 1, mini_batch_size: int = -1,
        do_update: bool = False, use_moun: bool = False, num_moun_iters: int = 3, weight_norm: bool = True):
    """ar_lact_swa_repeat.py:172-296: optional repeated update on the first mini-batch, then apply on all q."""
    mb = k.shape[1] if mini_batch_size == -1 else min(mini_batch_size, k.shape[1])
    steps = [(LACT_UPDATE, 0, mb, 0)] * (num_repeat if do_update else 0) + [(LACT_APPLY, 0, q.shape[1], 0)]
    prog = Program(steps=tuple(steps), out_len=q.shape[1],
                   ns_coeffs=(NS_CLASSIC,) * num_moun_iters if use_moun else None,
                   weight_norm=weight_norm, ns_mode=ops._ns_mode(q))
    out, ws, _ = run_program(prog, w0, w1, w2, q, k, v, _scaled(lr0, w_scale), _scaled(lr1, w_scale), _scaled(lr2, w_scale), None)
    return (out,) + tuple(ws)


def ar_fast_weight_swish_glu_weight_norm_mini_batch_inference_with_momentum(
        w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale: float, num_repeat: int = 1, mini_batch_size: int = -1,
        do_update: bool = False, use_moun: bool = False, num_moun_iters: int = 3, weight_norm: bool = True,
        fw_momentum: Optional[torch.Tensor] = None, dw0_momentum: Optional[torch.Tensor] = None,
        dw1_momentum: Optional[torch.Tensor] = None, dw2_momentum: Optional[torch.Tensor] = None,
        use_momentum: bool = False):
    """ar_lact_swa_repeat_sp.py:197-339.  Returns (output, w0, w1, w2, m0, m1, m2): the momentum states go in and
    come out, so that the caller can keep them between denoising steps.  Inference only (torch.no_grad)."""
    mb = k.shape[1] if mini_batch_size == -1 else min(mini_batch_size, k.shape[1])
    updates = num_repeat if do_update else 0
    steps = [(LACT_UPDATE, 0, mb, 0)] * updates + [(LACT_APPLY, 0, q.shape[1], 0)]
    prog = Program(steps=tuple(steps), out_len=q.shape[1],
                   ns_coeffs=(NS_CLASSIC,) * num_moun_iters if use_moun else None,
                   weight_norm=weight_norm, ns_mode=ops._ns_mode(q))
    state = (dw0_momentum, dw1_momentum, dw2_momentum) if (use_momentum and dw0_momentum is not None) else None
    out, ws, ms = run_program(prog, w0, w1, w2, q, k, v, _scaled(lr0, w_scale), _scaled(lr1, w_scale), _scaled(lr2, w_scale),
                              fw_momentum if use_momentum else None, momentum_state=state if updates else None)
    if not use_momentum:
        ms = (dw0_momentum, dw1_momentum, dw2_momentum)           # handed through untouched (:339)
    elif updates == 0 and state is not None:
        ms = state
    return (out,) + tuple(ws) + tuple(ms)


class FastWeightInferenceCache:
    """The fast-weight state a video layer keeps between denoising steps (ar_lact_swa_repeat.py:881-913,
    ar_lact_swa_repeat_sp.py:763-766,998-1053,1147-1148): one set of weights and momentum states for the
    conditional sequence and one for the classifier-free-guidance sequence, which take turns call by call.
    Both restart from the layer's parameters while no frame has been generated (`frame_offset == 0`) or one
    of the two sets does not exist yet; a set is replaced only by a call that updates (`do_update`)."""

    def __init__(self, use_momentum: bool = False):
        self.use_momentum = use_momentum
        self.reset()

    def reset(self):
        self.frame_offset = 0
        self.cfg_seq = False
        self.cur = None        # (w0, w1, w2, m0, m1, m2) of the conditional sequence
        self.cfg = None        # ... of the guidance sequence

    def step(self, w0, w1, w2, q, k, v, lr0, lr1, lr2, w_scale: float, *, do_update: bool, frames: int = 0,
             fw_momentum: Optional[torch.Tensor] = None, num_repeat: int = 1, mini_batch_size: int = -1,
             use_moun: bool = False, num_moun_iters: int = 3, weight_norm: bool = True) -> torch.Tensor:
        """One layer call: `w0, w1, w2` are the layer's parameters repeated over the batch, used when the cache
        restarts.  `frames` is the window length by which the conditional sequence advances on an updating call
        (:914-924).  Flips to the other sequence afterwards (:1147-1148).  Returns the output."""
        if do_update and not self.cfg_seq:
            self.frame_offset += frames
        fresh = self.cur is None or self.cfg is None or self.frame_offset == 0
        held = None if fresh else (self.cfg if self.cfg_seq else self.cur)
        ws = (w0, w1, w2) if held is None else held[:3]
        ms = (None, None, None) if held is None else held[3:]
        res = ar_fast_weight_swish_glu_weight_norm_mini_batch_inference_with_momentum(
            ws[0], ws[1], ws[2], q, k, v, lr0, lr1, lr2, w_scale, num_repeat, mini_batch_size, do_update, use_moun,
            num_moun_iters, weight_norm, fw_momentum, ms[0], ms[1], ms[2], self.use_momentum)
        if do_update:
            if self.cfg_seq:
                self.cfg = tuple(res[1:])
            else:
                self.cur = tuple(res[1:])
        self.cfg_seq = not self.cfg_seq
        return res[0]
