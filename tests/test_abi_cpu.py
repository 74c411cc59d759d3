"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares, and its
host-side validation and buffer sizing behave (no kernel is launched)."""
import ctypes
import os
import re

import pytest

from lact_amd import _lib, ops
from lact_amd._lib import LACT_APPLY, LACT_UPDATE
from oracle import lact_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "lact_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lact_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    names = header_functions()
    assert set(names) == set(_lib.EXPORTS)
    for n in names:
        assert getattr(L, n) is not None
    assert L.lact_version() >= 1


def make_desc(steps, b=2, d=64, dh=64, L=256, **kw):
    arr = (_lib.Step * len(steps))(*[_lib.Step(*s) for s in steps])
    D = _lib.Desc()
    D.b, D.d, D.dh, D.q_len, D.kv_len, D.out_len = b, d, dh, L, L, L
    D.act_dtype, D.n_steps, D.steps = 0, len(steps), ctypes.cast(arr, ctypes.POINTER(_lib.Step))
    D.ns_steps, D.weight_norm = -1, 1
    for name in ("q", "k", "v", "o", "do"):
        setattr(D, name + "_ld", d)
        setattr(D, name + "_bs", L * d)
    for k_, v_ in kw.items():
        setattr(D, k_, v_)
    D._keep = arr
    return D


def sizes(D):
    a, s = ctypes.c_size_t(0), ctypes.c_size_t(0)
    rc = _lib.lib().lact_query_sizes(ctypes.byref(D), ctypes.byref(a), ctypes.byref(s))
    return rc, a.value, s.value


def test_query_sizes_and_validation_messages():
    L = _lib.lib()
    ok = make_desc(ops.block_causal_steps(256, 64))
    rc, saved, scratch = sizes(ok)
    assert rc == 0 and saved > 0 and scratch > 0
    # more updates -> more saved state; Muon adds the Newton-Schulz iterates
    rc, saved2, _ = sizes(make_desc(ops.block_causal_steps(256, 32)))
    assert rc == 0 and saved2 > saved
    coeffs = (ctypes.c_float * 15)(*[x for t in ops.NS5_COEFFS for x in t])
    rc, saved3, _ = sizes(make_desc(ops.block_causal_steps(256, 64), ns_steps=5,
                                    ns_coeffs=ctypes.cast(coeffs, ctypes.POINTER(ctypes.c_float))))
    assert rc == 0 and saved3 > saved

    def err(D):
        rc, _, _ = sizes(D)
        assert rc != 0
        return L.lact_last_error().decode()

    assert "multiples of 8" in err(make_desc(ops.block_causal_steps(256, 64), d=60))
    assert "exceeds kv_len" in err(make_desc(((LACT_UPDATE, 0, 300, 0),)))
    assert "exceeds q_len" in err(make_desc(((LACT_APPLY, 0, 300, 0),)))
    assert "out_len" in err(make_desc(((LACT_APPLY, 0, 256, 8),)))
    assert "empty" in err(make_desc(((LACT_APPLY, 5, 5, 0),)))
    assert "kind" in err(make_desc(((7, 0, 5, 0),)))
    assert "ns_coeffs" in err(make_desc(ops.block_causal_steps(256, 64), ns_steps=5))
    assert "alignment" in err(make_desc(ops.block_causal_steps(256, 64), q_ld=68))
    assert "act_dtype" in err(make_desc(ops.block_causal_steps(256, 64), act_dtype=3))
    # a forward-only descriptor keeps less for the backward, and the backward entry point refuses it (before it
    # looks at any pointer: no GPU is needed for this check)
    # (at d = 256: the update's pre-activations are kept for the backward only above d = 128)
    rc, saved_bw, _ = sizes(make_desc(ops.block_causal_steps(256, 64), d=256, dh=256))
    rc_fo, saved_fo, _ = sizes(make_desc(ops.block_causal_steps(256, 64), d=256, dh=256, forward_only=1))
    assert rc == 0 and rc_fo == 0 and saved_fo < saved_bw
    null = ctypes.c_void_p(0)
    fo = make_desc(ops.block_causal_steps(256, 64), forward_only=1)
    assert L.lact_backward(ctypes.byref(fo), *([null] * 22)) != 0
    assert "forward_only" in L.lact_last_error().decode()
    # a carried momentum state is an inference feature: needs use_momentum and forward_only, and costs one more
    # state array in `saved`
    assert "momentum_state_in" in err(make_desc(ops.block_causal_steps(256, 64), momentum_state_in=1, use_momentum=1))
    assert "momentum_state_in" in err(make_desc(ops.block_causal_steps(256, 64), momentum_state_in=1, forward_only=1))
    rc, saved_mo, _ = sizes(make_desc(ops.block_causal_steps(256, 64), forward_only=1, use_momentum=1))
    rc2, saved_st, _ = sizes(make_desc(ops.block_causal_steps(256, 64), forward_only=1, use_momentum=1, momentum_state_in=1))
    assert rc == 0 and rc2 == 0 and saved_st > saved_mo
    assert L.lact_query_sizes(None, None, None) != 0 and "null" in L.lact_last_error().decode()
    assert L.lact_newton_schulz_workspace_bytes(4, 64, 128, 5) > 0
    assert L.lact_newton_schulz_workspace_bytes(0, 64, 128, 5) == 0


@pytest.mark.parametrize("L,C", [(64, 16), (70, 16), (16, 16), (10, 16), (17, 16), (4096, 2048), (32760, 4680)])
def test_schedule_builder_matches_oracle(L, C):
    mine = ops.block_causal_steps(L, C)
    ref = O.block_causal_steps(L, C)
    assert [(s[0], s[1], s[2]) for s in mine] == [(0 if s.kind == O.UPDATE else 1, s.start, s.end) for s in ref]
    assert all(s[3] == s[1] for s in mine if s[0] == LACT_APPLY)


def test_ar_video_schedule_matches_oracle():
    """The video step lists against the oracle's, which the oracle tests pin against the reference's loop bounds: the
    documented case and 300 random argument sets (defaults by -1, cut last windows, updates that stop early,
    repeats).  The oracle slices tensors (a range past the end is cut there); the builder states the cut ranges."""
    import numpy as np
    from lact_amd import ar_video
    cases = [(60, 10, 60, 20, 2)]
    rng = np.random.default_rng(7)
    for _ in range(300):
        L = int(rng.integers(8, 400))
        mb = int(rng.choice([-1, int(rng.integers(1, L + 1))]))
        ul = int(rng.choice([-1, int(rng.integers(1, L + 1))]))
        eff_mb = (L if ul == -1 else ul) if mb == -1 else mb
        ue = int(rng.choice([-1, eff_mb + int(rng.integers(1, L + 40))]))      # the first window may exceed the sequence
        cases.append((L, mb, ul, ue, int(rng.integers(1, 4))))
    for L, mb, ul, ue, rep in cases:
        mine = ar_video._ar_steps(L, L, mb, ul, ue, rep)
        ref = O.ar_video_steps(L, mb, ul, ue, rep)
        cut = [(0 if s.kind == O.UPDATE else 1, min(s.start, L), min(s.end, L)) for s in ref]
        assert [(s[0], s[1], s[2]) for s in mine] == cut, (L, mb, ul, ue, rep)
        assert all(s[2] > s[1] for s in mine), (L, mb, ul, ue, rep)      # no empty range reaches the library


def test_cpu_tensors_are_refused():
    import torch
    w = torch.zeros(1, 8, 8)
    x = torch.zeros(1, 4, 8)
    lr = torch.zeros(1, 4, 1)
    with pytest.raises(RuntimeError, match="no CPU path"):
        from lact_amd import block_causal_lact_swiglu
        block_causal_lact_swiglu(w, w, w, x, x, x, lr, lr, lr, 2)
