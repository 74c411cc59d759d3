"""GPU parity: the HIP path (through liblact_hip.so's C ABI) against the CPU oracle on the same seeded
inputs.

Tolerances (relative L2, written where they are used):
  * fp32 activations, Muon off ................................ 1e-4   (north-star fp32 bound)
  * fp32 activations, Newton-Schulz in fp32 (LACT_NS_FP32) ..... 1e-3   against float64 arithmetic; checks the
                                                                closed-form Muon forward/backward itself
  * bf16 activations, Muon off ................................ 1e-2   (north-star bf16 bound)
  * bf16 Newton-Schulz (Muon on): the HIP path rounds at the reference's own rounding points (every tensor
    of the eager autocast flow is a rounding point; the no-autocast Newton-Schulz comes out bit-identical to the
    oracle at several shapes below), but the iteration amplifies single bf16 rounding flips to percent level, and
    which values flip depends on the order in which a GEMM or a sum of squares adds its terms -- which no two
    libraries share.  The yardstick is therefore the ORDER-ONLY FLOOR: the oracle against itself with nothing
    changed but that order (O.order_variants: float64 accumulation, K blocks of 16 ascending, K blocks of 64
    descending; tests/test_oracle_pins.py pins its size, about 1e-2 on the output).  Bound:
      err(HIP, oracle) <= 1.5 * max over variants err(variant, oracle) + 1e-3.
"""
import math
import os
import sys

import numpy as np
import pytest
import torch

from lact_amd import ar_video, minimal, nvs, ops
from lact_amd import ttt_operation as T
from lact_amd._lib import LACT_APPLY
from oracle import lact_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
AC = O.Numerics(autocast=True)
PLAIN = O.Numerics(autocast=False)
EXACT = O.Numerics(autocast=False, ns_dtype=None)
NAMES = ["w0", "w1", "w2", "q", "k", "v", "lr0", "lr1", "lr2", "momentum"]


def say(*a):
    print(*a)
    sys.stdout.flush()


def problem(b, L, d, dh, seed, act, momentum=True, lr_shift=-3.0, lr_scale=1.0):
    inp = O.make_inputs(b, L, d, dh, seed=seed, act_dtype=act, lr_shift=lr_shift, lr_scale=lr_scale,
                        momentum_value=None)
    if momentum:
        g = torch.Generator().manual_seed(seed + 99)
        inp["momentum"] = torch.sigmoid(torch.randn(b, L, 1, generator=g) + 1.5)
    return inp


def clone_to(inp, device, dtype_map=None, grad=True):
    out = {}
    for n, t in inp.items():
        if t is None:
            out[n] = None
            continue
        t = t.detach().clone()
        if dtype_map is not None:
            t = t.to(dtype_map(t))
        t = t.to(device)
        out[n] = t.requires_grad_(grad)
    return out


def grads_of(out, inp, go):
    names = [n for n in NAMES if inp.get(n) is not None]
    gs = torch.autograd.grad(out, [inp[n] for n in names], go, allow_unused=True)
    return {n: g for n, g in zip(names, gs)}


def compare(res, ref):
    return {n: O.rel_l2(res[n], ref[n]) for n in ref if ref[n] is not None and float(ref[n].double().norm()) > 0}


def run_both(hip_fn, oracle_fn, inp, num, upstream_seed=3, ref64=False, floor=False):
    """Returns (hip results, oracle results [, float64 results] [, order-only floors]) as dicts: out + every gradient."""
    g = clone_to(inp, DEV)
    out = hip_fn(g)
    go = torch.randn(out.shape, generator=torch.Generator().manual_seed(upstream_seed))
    res = {"out": out, **grads_of(out, g, go.to(out.dtype).to(DEV))}
    torch.cuda.synchronize()

    def oracle_run(numerics, dtype_map=None):
        c = clone_to(inp, "cpu", dtype_map=dtype_map)
        o = oracle_fn(c, numerics)
        return {"out": o, **grads_of(o, c, go.to(o.dtype))}
    ret = [res, oracle_run(num)]
    if ref64:
        ret.append(oracle_run(EXACT, lambda t: torch.float64))
    if floor:
        ret.append(order_floor(oracle_run, num, ret[1]))
    return tuple(ret)


def order_floor(oracle_run, num, ref):
    """Largest distance of the oracle from itself when only the accumulation order of its GEMMs and norms changes."""
    floors = {}
    for v in O.order_variants(num):
        for n, e in compare(oracle_run(v), ref).items():
            floors[n] = max(floors.get(n, 0.0), e)
    return floors


def assert_within_order_floor(res, ref, floors, label, r64=None, factor=1.5, slack=1e-3):
    """r64 (the float64 oracle): only for the entry `momentum`.  d loss / d momentum is <g, M_prev> per head and update,
    a handful of numbers, and g is orthogonal to the Newton-Schulz input dw + m M_prev in exact arithmetic (the
    iteration is scale invariant), so what is left is a small difference that magnifies the rounding of the backward
    pass: its yardstick is the larger of the order-only floor and the oracle's own distance from float64, and, being a
    relative error over four to eight numbers, it gets a factor of 2 instead of 1.5."""
    e_ref = compare(res, ref)
    yard = dict(floors)
    if r64 is not None and "momentum" in e_ref:
        yard["momentum"] = max(yard["momentum"], O.rel_l2(ref["momentum"], r64["momentum"]))
    for n in e_ref:
        say(f"   {label} {n:9s} hip-vs-oracle {e_ref[n]:.4f}  order-only floor {floors[n]:.4f}  ratio {e_ref[n] / max(yard[n], 1e-12):.2f}")
    for n in e_ref:
        assert e_ref[n] <= (2.0 if n == "momentum" else factor) * yard[n] + slack, (n, e_ref[n], yard[n])


def args9(t):
    return (t["w0"], t["w1"], t["w2"], t["q"], t["k"], t["v"], t["lr0"], t["lr1"], t["lr2"])


# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("b,L,d,dh,act,tol", [
    (2, 200, 64, 64, torch.bfloat16, 1e-3), (3, 333, 128, 256, torch.bfloat16, 1e-3),
    (2, 300, 384, 384, torch.bfloat16, 1e-3), (1, 7, 8, 16, torch.bfloat16, 1e-3),
    (2, 200, 64, 64, torch.float32, 1e-5), (2, 130, 128, 256, torch.float32, 1e-5), (1, 5, 24, 8, torch.float32, 1e-5)])
def test_apply_only(b, L, d, dh, act, tol):
    say("apply_only", b, L, d, dh, act)
    inp = problem(b, L, d, dh, 1, act, momentum=False)
    prog = ops.Program(steps=((LACT_APPLY, 0, L, 0),), out_len=L)
    g = clone_to(inp, DEV, grad=False)
    out, wfin, _ = ops.run_program(prog, g["w0"], g["w1"], g["w2"], g["q"], None, None, None, None, None, None)
    ref = O.swiglu_apply(inp["w0"], inp["w1"], inp["w2"], inp["q"], AC if act == torch.bfloat16 else PLAIN)
    assert out.dtype == act and O.rel_l2(out, ref) < tol
    assert torch.equal(wfin[0].cpu(), inp["w0"])          # no update: weights come back untouched


@pytest.mark.parametrize("n,r,c,kind,steps", [(4, 64, 64, "llm", 5), (3, 128, 256, "llm", 5), (3, 256, 128, "classic", 3),
                                              (2, 384, 384, "llm", 5), (2, 64, 128, "classic", 0), (2, 40, 24, "classic", 5)])
def test_newton_schulz_standalone(n, r, c, kind, steps):
    say("newton_schulz", n, r, c, kind, steps)
    G = torch.randn(n, r, c, generator=torch.Generator().manual_seed(5))
    co = O.ns_coeff_table(kind, steps)
    ref64 = O.newton_schulz(G.double(), co, EXACT)
    # exact mode: the iteration itself
    out = ops.newton_schulz(G.to(DEV), co, ns_mode=ops.NS_FP32)
    e = O.rel_l2(out, ref64)
    say("   fp32 mode vs float64:", e)
    assert out.dtype == torch.float32 and e < 1e-3
    # reference numerics (with and without autocast) against the oracle's, bounded by the order-only floor
    for label, num, mode, dtype in (("autocast", AC, ops.NS_AUTOCAST, torch.float32), ("plain", PLAIN, ops.NS_PLAIN_BF16, torch.bfloat16)):
        ref = O.newton_schulz(G, co, num)
        floor = max(O.rel_l2(O.newton_schulz(G, co, v), ref) for v in O.order_variants(num))
        out = ops.newton_schulz(G.to(DEV), co, ns_mode=mode)
        e_ref = O.rel_l2(out, ref)
        say(f"   {label}: vs oracle {e_ref:.5f}  order-only floor {floor:.5f}  (oracle vs f64 {O.rel_l2(ref, ref64):.4f})")
        assert out.dtype == dtype
        assert e_ref <= 1.5 * floor + 1e-3


@pytest.mark.parametrize("n,r,c,kind,steps", [(3, 64, 64, "llm", 5), (2, 128, 256, "llm", 5), (2, 256, 128, "classic", 3),
                                              (2, 384, 384, "llm", 5), (2, 40, 24, "classic", 2), (2, 64, 128, "classic", 0)])
def test_newton_schulz_standalone_is_differentiable(n, r, c, kind, steps):
    """zeropower_via_newtonschulz5 is an ordinary differentiable function in the reference (ttt_operation.py:30-66):
    lact_newton_schulz_backward against autograd through the oracle.  fp32 mode against float64 pins the closed form;
    the reference's numerics are held to the larger of the order-only floor and the oracle's own distance from
    float64 (the closed-form backward rounds at other points than autograd does: another realisation of the same
    bf16 noise)."""
    say("newton_schulz backward", n, r, c, kind, steps)
    gen = torch.Generator().manual_seed(23)
    G, go = torch.randn(n, r, c, generator=gen), torch.randn(n, r, c, generator=gen)
    co = O.ns_coeff_table(kind, steps)

    def oracle_grad(num, dt):
        x = G.to(dt).requires_grad_(True)
        y = O.newton_schulz(x, co, num)
        return torch.autograd.grad(y, x, go.to(y.dtype))[0]

    def hip_grad(mode):
        x = G.to(DEV).requires_grad_(True)
        y = ops.newton_schulz(x, co, ns_mode=mode)
        return torch.autograd.grad(y, x, go.to(DEV).to(y.dtype))[0]
    g64 = oracle_grad(EXACT, torch.float64)
    e = O.rel_l2(hip_grad(ops.NS_FP32), g64)
    say("   fp32 mode vs float64:", e)
    assert e < 1e-3
    for label, num, mode in (("autocast", AC, ops.NS_AUTOCAST), ("plain", PLAIN, ops.NS_PLAIN_BF16)):
        ref = oracle_grad(num, torch.float32)
        yard = max([O.rel_l2(ref, g64)] + [O.rel_l2(oracle_grad(v, torch.float32), ref) for v in O.order_variants(num)])
        e = O.rel_l2(hip_grad(mode), ref)
        say(f"   {label}: vs oracle {e:.4f}  yardstick {yard:.4f}")
        assert e <= 1.5 * yard + 1e-3


def test_no_grad_with_parameters_runs_the_inference_descriptor():
    """Under torch.no_grad() inputs that require a gradient (nn.Parameter fast weights) still make autograd report
    needs_input_grad; the call must all the same take the forward-only path -- smaller buffers, and the carried
    momentum state (an inference feature) accepted."""
    say("no_grad with requires_grad inputs")
    inp = problem(2, 3 * 64, 64, 128, 31, torch.bfloat16, momentum=True)
    g = clone_to(inp, DEV)                                    # every tensor requires a gradient
    prog = ops.Program(steps=ops.block_causal_steps(3 * 64, 64), out_len=3 * 64, ns_coeffs=O.NS5_COEFFS)
    with torch.no_grad():
        out, ws, ms = ops.run_program(prog, *args9(g), g["momentum"])
        M = [m.clone() for m in ms]
        out2, _, ms2 = ops.run_program(prog, *args9(g), g["momentum"], momentum_state=M)     # raised before the fix
    assert not out.requires_grad and torch.isfinite(out.float()).all() and torch.isfinite(out2.float()).all()
    ref, _, _ = ops.run_program(prog, *args9(g), g["momentum"])                              # training descriptor
    assert ref.requires_grad and torch.equal(ref.detach(), out)
    assert not torch.equal(ms2[0], ms[0])                     # the carried state was used


def block_causal_pair(C, use_muon, prenorm=False):
    fn = T.prenorm_block_causal_lact_swiglu if prenorm else T.block_causal_lact_swiglu
    hip = lambda t: fn(*args9(t), C, use_muon, t["momentum"])
    orc = lambda t, num: O.block_causal_lact_swiglu(*args9(t), C, use_muon, t["momentum"], num=num, prenorm=prenorm)
    return hip, orc


@pytest.mark.parametrize("b,L,d,dh,C,mom,prenorm", [
    (2, 3 * 64 + 5, 64, 64, 64, False, False), (2, 3 * 64 + 5, 64, 64, 64, True, False),
    (2, 2 * 96 + 17, 64, 128, 96, True, False), (2, 2 * 96 + 17, 128, 64, 96, True, True),
    (3, 4 * 200, 384, 384, 200, True, False), (1, 100, 64, 64, 128, True, False),
    (2, 2 * 96 + 17, 40, 136, 96, True, False),    # d not a multiple of 64: generic tile kernels, two hidden tiles
    (2, 2 * 96 + 17, 64, 192, 96, True, False),    # dh = 128 + 64: a half-valid hidden tile on the asynchronous-copy path
    (2, 2 * 3200 + 100, 64, 64, 3200, True, False)])   # long chunks, few tiles: token reductions split in two, partial sums
def test_block_causal_bf16_no_muon(b, L, d, dh, C, mom, prenorm):
    say("block_causal bf16 no muon", b, L, d, dh, C, mom, prenorm)
    inp = problem(b, L, d, dh, 7, torch.bfloat16, momentum=mom)
    res, ref = run_both(*block_causal_pair(C, False, prenorm), inp, AC)
    errs = compare(res, ref)
    say("  ", errs)
    assert res["out"].dtype == torch.bfloat16
    # the forward rounds where the reference rounds: output and (through them) the fast-weight states agree up to
    # the summation order inside the GEMMs
    assert errs["out"] < 1e-3
    for n, e in errs.items():
        assert e < 1e-2, n                             # north-star bf16 bound


@pytest.mark.parametrize("b,L,d,dh,C,mom,prenorm", [
    (2, 3 * 64 + 5, 64, 64, 64, True, False), (2, 2 * 96 + 17, 64, 128, 96, True, True),
    (2, 2 * 96 + 17, 128, 64, 96, False, False), (2, 2 * 96 + 17, 40, 136, 96, True, False),
    (2, 2 * 3100 + 50, 64, 64, 3100, True, False)])    # split token reductions on the generic kernels
def test_block_causal_fp32_no_muon(b, L, d, dh, C, mom, prenorm):
    say("block_causal fp32 no muon", b, L, d, dh, C, mom, prenorm)
    inp = problem(b, L, d, dh, 8, torch.float32, momentum=mom)
    res, ref = run_both(*block_causal_pair(C, False, prenorm), inp, PLAIN)
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < 1e-4                       # north-star fp32 bound


@pytest.mark.parametrize("b,L,d,dh,C,mom,prenorm", [
    (2, 3 * 64 + 5, 64, 64, 64, True, False), (2, 2 * 96 + 17, 64, 128, 96, True, False),
    (2, 2 * 96 + 17, 128, 64, 96, True, True), (2, 3 * 128, 384, 384, 128, True, False)])
def test_block_causal_muon_exact_arithmetic(b, L, d, dh, C, mom, prenorm):
    """fp32 activations + fp32 Newton-Schulz against float64: pins the Muon forward and its hand-derived
    backward (momentum carry, Frobenius normalisation, quintic iteration, renorm) without bf16 noise."""
    say("block_causal exact muon", b, L, d, dh, C, mom, prenorm)
    inp = problem(b, L, d, dh, 9, torch.float32, momentum=mom, lr_shift=-1.0)
    hip, orc = block_causal_pair(C, True, prenorm)

    def hip_exact(t):
        with ops.newton_schulz_mode(ops.NS_FP32):
            return hip(t)
    g = clone_to(inp, DEV)
    out = hip_exact(g)
    go = torch.randn(out.shape, generator=torch.Generator().manual_seed(3))
    res = {"out": out, **grads_of(out, g, go.to(DEV))}
    c64 = clone_to(inp, "cpu", dtype_map=lambda t: torch.float64)
    o64 = orc(c64, EXACT)
    ref = {"out": o64, **grads_of(o64, c64, go.double())}
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < 1e-3


@pytest.mark.parametrize("b,L,d,dh,C,mom,prenorm", [
    (2, 3 * 64 + 5, 64, 64, 64, True, False), (2, 2 * 96 + 17, 64, 128, 96, True, False),
    (2, 2 * 96 + 17, 128, 64, 96, False, True), (4, 1024, 384, 384, 512, True, False)])
def test_block_causal_bf16_muon(b, L, d, dh, C, mom, prenorm):
    say("block_causal bf16 muon", b, L, d, dh, C, mom, prenorm)
    inp = problem(b, L, d, dh, 7, torch.bfloat16, momentum=mom)
    res, ref, r64, floors = run_both(*block_causal_pair(C, True, prenorm), inp, AC, ref64=True, floor=True)
    assert_within_order_floor(res, ref, floors, "bf16-muon", r64)


def test_minimal_argument_order_and_short_sequence():
    say("minimal arg order / L <= C")
    inp = problem(2, 150, 64, 64, 11, torch.bfloat16)
    g = clone_to(inp, DEV, grad=False)
    a = T.block_causal_lact_swiglu(*args9(g), 64, True, g["momentum"])
    b_ = minimal.block_causal_lact_swiglu(*args9(g), g["momentum"], True, 64)
    assert torch.equal(a, b_)                               # same program, deterministic kernels
    short = T.block_causal_lact_swiglu(*args9(g), 256, True, g["momentum"])       # L <= C: apply only
    ref = O.swiglu_apply(inp["w0"], inp["w1"], inp["w2"], inp["q"], AC)
    assert O.rel_l2(short, ref) < 1e-3


def test_strided_inputs_and_per_token_shapes():
    say("strided q/k/v views")
    b, L, d, dh = 2, 160, 64, 128
    inp = problem(b, L, d, dh, 12, torch.bfloat16)
    g = clone_to(inp, DEV, grad=False)
    packed = torch.cat([g["q"], g["k"], g["v"]], dim=-1)              # [b, L, 3d]
    qv, kv, vv = packed.split(d, dim=-1)                              # row stride 3d, not contiguous
    assert not qv.is_contiguous()
    a = T.block_causal_lact_swiglu(g["w0"], g["w1"], g["w2"], qv, kv, vv, g["lr0"], g["lr1"], g["lr2"], 64, True, g["momentum"])
    b_ = T.block_causal_lact_swiglu(*args9(g), 64, True, g["momentum"])
    assert torch.equal(a, b_)
    with pytest.raises(ValueError, match="one value per head and token"):
        T.block_causal_lact_swiglu(g["w0"], g["w1"], g["w2"], g["q"], g["k"], g["v"], g["lr0"].expand(b, L, d),
                                   g["lr1"], g["lr2"], 64)


# ---- bidirectional layer op (config 0) -------------------------------------------------------------
def bidirectional_pair(use_muon, mode="reference"):
    hip = lambda t: minimal.bidirectional_lact_swiglu(*args9(t), use_muon, muon_mode=mode)
    orc = lambda t, num: O.bidirectional_lact_swiglu(*args9(t), use_muon, num=num, muon_mode=mode)
    return hip, orc


def c0_inputs(b=2, L=1024, d=64, dh=64):
    return O.make_inputs(b, L, d, dh, seed=1000, act_dtype=torch.float32, lr_shift=0.0, lr_scale=1e-2,
                         momentum_value=None, normalize_v=True)


def test_bidirectional_config0_fp32():
    """BASELINE config 0: fp32, b=2, 1024 tokens, d=dh=64, Muon.  Without Muon the fp32 bound (1e-4) holds
    outright; with Muon the reference itself runs Newton-Schulz in bf16, so the noise-floor bound applies,
    and the exact-arithmetic mode is held to 1e-3 of float64."""
    say("bidirectional c0 fp32")
    inp = c0_inputs()
    res, ref = run_both(*bidirectional_pair(False), inp, PLAIN)
    errs = compare(res, ref)
    say("   no muon", errs)
    assert max(errs.values()) < 1e-4
    res, ref, floors = run_both(*bidirectional_pair(True), inp, PLAIN, floor=True)
    assert res["out"].dtype == torch.float32
    assert_within_order_floor(res, ref, floors, "c0-muon")
    hip, orc = bidirectional_pair(True)

    def hip_exact(t):
        with ops.newton_schulz_mode(ops.NS_FP32):
            return hip(t)
    res, _, r64 = run_both(hip_exact, orc, inp, PLAIN, ref64=True)
    errs = compare(res, r64)
    say("   exact muon", errs)
    assert max(errs.values()) < 1e-3
    # "intended" Muon (w + NS(dw)) is a different function
    res_i, ref_i = run_both(*bidirectional_pair(True, "intended"), inp, PLAIN)
    assert O.rel_l2(res_i["out"], res["out"]) > 1e-2


@pytest.mark.parametrize("tag", ["muon", "nomuon", "square"])
def test_bidirectional_golden_vectors(tag):
    """Vectors written from the reference itself on the CPU (tests/golden/make_bidirectional_golden.py)."""
    say("bidirectional golden", tag)
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "bidirectional_muon_cpu_fp32.npz"))
    t = {n: torch.from_numpy(z[f"{tag}.{n}"]) for n in ("w0", "w1", "w2", "q", "k", "v", "lr0", "lr1", "lr2", "o")}
    use_muon = bool(z[f"{tag}.use_muon"])
    g = {n: v.to(DEV) for n, v in t.items()}
    out = minimal.bidirectional_lact_swiglu(*args9(g), use_muon)
    e = O.rel_l2(out, t["o"])
    if not use_muon:
        say("   vs reference", e)
        assert e < 1e-4
        return
    # the vectors are the reference's own CPU run: the oracle's order variants give the floor around it
    ref = O.bidirectional_lact_swiglu(*args9(t), True, num=PLAIN)
    floor = max(O.rel_l2(O.bidirectional_lact_swiglu(*args9(t), True, num=v), ref) for v in O.order_variants(PLAIN))
    say("   vs reference", e, "order-only floor", floor, "oracle vs reference", O.rel_l2(ref, t["o"]))
    assert e <= 1.5 * floor + 1e-3


# ---- golden vectors of the LLM operations and the NVS program, written from the reference (CPU, fp32) ------------
from test_oracle_pins import LLM_TAGS, NVS_TAGS, load_llm_nvs_gold, run_oracle_on_gold  # noqa: E402


@pytest.mark.parametrize("tag", LLM_TAGS + NVS_TAGS)
def test_llm_and_nvs_golden_vectors(tag):
    """tests/golden/make_llm_nvs_golden.py: the reference's own block_causal_lact_swiglu /
    prenorm_block_causal_lact_swiglu (ttt_operation.py:71-364) and NVS program (lact_ttt.py:71-147) on the CPU in
    fp32: outputs, returned weights and the gradient of every input.  Without Newton-Schulz the fp32 bound holds;
    with it (bf16 on both sides) the order-only floor around the reference's vectors is the yardstick."""
    say("llm / nvs golden", tag)
    t, outs, gos, grads, meta = load_llm_nvs_gold(tag)
    g = {n: v.to(DEV).requires_grad_(True) for n, v in t.items()}
    if tag.startswith("llm"):
        fn = T.prenorm_block_causal_lact_swiglu if bool(meta["prenorm"]) else T.block_causal_lact_swiglu
        res = [fn(*args9(g), int(meta["chunk"]), bool(meta["use_muon"]), g.get("momentum"))]
        bf16_ns = bool(meta["use_muon"])
    else:
        order = [nvs.TTTOperator(int(s0), int(e0), bool(u), bool(ap)) for s0, e0, u, ap in meta["order"]]
        res = list(nvs.fast_weight_swish_glu_weight_norm_mini_batch_apply(*args9(g), order, int(meta["steps"])))
        bf16_ns = True           # lact_ttt.py:117-126 casts to bf16 and normalises even with zero iterations
    loss = sum((r.float() * go.to(DEV)).sum() for r, go in zip(res, gos))
    names = list(grads)
    got = dict(zip(names, torch.autograd.grad(loss, [g[n] for n in names])))
    errs = {f"out{i}": O.rel_l2(r, o) for i, (r, o) in enumerate(zip(res, outs))}
    errs.update({n: O.rel_l2(got[n], grads[n]) for n in names if float(grads[n].norm()) > 0})
    say("  ", {n: float("%.2e" % e) for n, e in errs.items()})
    if not bf16_ns:
        assert max(errs.values()) < 1e-4
        return
    yard = {n: 0.0 for n in errs}
    for v in O.order_variants(PLAIN):
        tt, r = run_oracle_on_gold(tag, t, meta, num=v)
        l = sum((x.float() * go).sum() for x, go in zip(r, gos))
        gv = dict(zip(names, torch.autograd.grad(l, [tt[n] for n in names])))
        for i, (x, o) in enumerate(zip(r, outs)):
            yard[f"out{i}"] = max(yard[f"out{i}"], O.rel_l2(x, o))
        for n in names:
            if n in yard:
                yard[n] = max(yard[n], O.rel_l2(gv[n], grads[n]))
    say("   order-only floor", {n: float("%.2e" % e) for n, e in yard.items()})
    # Gradients pass through the backward of the bf16 iteration, where the closed-form HIP backward rounds each of its
    # three products per iteration once and autograd rounds every partial product and every gradient accumulation:
    # as many roundings at other points, i.e. another realisation of the same noise.  On matrices this small the
    # forward comes out without a single flip (outputs and weights above agree to fp32 round-off) and the order-only
    # floor is far below that noise, so for the gradients the yardstick is the larger of the floor and the distance
    # of the reference's own vectors from float64 arithmetic.
    t64, r64 = run_oracle_on_gold(tag, {n: v.double() for n, v in t.items()}, meta, num=EXACT)
    l64 = sum((x * go.double()).sum() for x, go in zip(r64, gos))
    g64 = dict(zip(names, torch.autograd.grad(l64, [t64[n] for n in names])))
    for n in names:
        if n in yard:
            yard[n] = max(yard[n], O.rel_l2(grads[n], g64[n]))
    say("   gradient yardstick", {n: float("%.2e" % yard[n]) for n in names if n in yard})
    for n, e in errs.items():
        assert e <= (2.0 if n == "momentum" else 1.5) * yard[n] + 1e-3, (n, e, yard[n])


# ---- NVS program (config 3 shape family) -----------------------------------------------------------
def test_nvs_program_returns_weights_and_grads():
    say("nvs program")
    b, d, dh, n_in, n_tgt = 2, 64, 128, 256, 96
    L = n_in + n_tgt
    inp = problem(b, L, d, dh, 13, torch.bfloat16, momentum=False)
    # NVS layout: w0, w2 [b, d, dh]; w1 [b, dh, d]
    for n in ("w0", "w1", "w2"):
        inp[n] = inp[n].transpose(1, 2).contiguous()
    order = [nvs.TTTOperator(0, n_in, True, False), nvs.TTTOperator(0, L, False, True)]

    def hip(t):
        o, a0, a1, a2 = nvs.fast_weight_swish_glu_weight_norm_mini_batch_apply(*args9(t), order, 5)
        hip.extra = (a0, a1, a2)
        return o

    def orc(t, num):
        o, a0, a1, a2 = O.fast_weight_swish_glu_weight_norm_mini_batch_apply(*args9(t), order, 5, num=num)
        orc.extra = (a0, a1, a2)
        return o
    res, ref, floors = run_both(hip, orc, inp, AC, floor=True)
    assert res["out"].shape == (b, L, d) and hip.extra[0].shape == (b, d, dh) and hip.extra[1].shape == (b, dh, d)
    assert_within_order_floor(res, ref, floors, "nvs")
    # zero Newton-Schulz steps (normalisation only) and a gradient arriving through the returned weights
    g = clone_to(inp, DEV)
    o, a0, a1, a2 = nvs.fast_weight_swish_glu_weight_norm_mini_batch_apply(*args9(g), [nvs.TTTOperator(0, n_in, True, True)], 0)
    loss = (o.float() ** 2).sum() + (a0 * a0).sum() + a1.sum() + (a2 ** 3).sum()
    gh = torch.autograd.grad(loss, [g["w0"], g["w1"], g["k"], g["lr1"]])
    c = clone_to(inp, "cpu", dtype_map=lambda t: torch.float64)
    o, a0, a1, a2 = O.fast_weight_swish_glu_weight_norm_mini_batch_apply(*args9(c), [O.TTTOperator(0, n_in, True, True)], 0, num=EXACT)
    loss = (o ** 2).sum() + (a0 * a0).sum() + a1.sum() + (a2 ** 3).sum()
    gr = torch.autograd.grad(loss, [c["w0"], c["w1"], c["k"], c["lr1"]])
    errs = [O.rel_l2(x, y) for x, y in zip(gh, gr)]
    say("   steps=0 + weight-output grads", errs)
    assert max(errs) < 2e-2


def test_nvs_config3_shape_forward():
    """BASELINE config 3 at full size: update on 8192 tokens, apply on 1024, d=128, dh=256, forward only."""
    say("nvs config 3")
    b, d, dh = 6, 128, 256
    inp = O.make_inputs(b, 9216, d, dh, seed=1003, act_dtype=torch.bfloat16, momentum_value=None)
    for n in ("w0", "w1", "w2"):
        inp[n] = (inp[n] * math.sqrt(2.0)).transpose(1, 2).contiguous()
    order = [nvs.TTTOperator(0, 8192, True, False), nvs.TTTOperator(8192, 9216, False, True)]
    g = clone_to(inp, DEV, grad=False)
    out, a0, a1, a2 = nvs.fast_weight_swish_glu_weight_norm_mini_batch_apply(*args9(g), order, 5)
    run = lambda num: O.fast_weight_swish_glu_weight_norm_mini_batch_apply(*args9(inp), order, 5, num=num)
    ref, r0, r1, r2 = run(AC)
    names = ("out", "w0", "w1", "w2")
    floors = {n: 0.0 for n in names}
    for v in O.order_variants(AC):
        for n, x, y in zip(names, run(v), (ref, r0, r1, r2)):
            floors[n] = max(floors[n], O.rel_l2(x, y))
    assert out.shape == (b, 1024, d)
    for n, x, y in zip(names, (out, a0, a1, a2), (ref, r0, r1, r2)):
        e = O.rel_l2(x, y)
        say(f"   {n}: hip-vs-oracle {e:.5f}  order-only floor {floors[n]:.5f}")
        assert e <= 1.5 * floors[n] + 1e-3, n


# ---- AR-video schedule -----------------------------------------------------------------------------
@pytest.mark.parametrize("use_momentum,weight_norm,use_moun,repeat", [
    (False, True, True, 1), (True, False, False, 1), (True, True, True, 1),
    (True, True, False, 2)])      # every chunk updated twice: k, v, lr and momentum gradients of a chunk add up
@pytest.mark.parametrize("L,update_length", [(240, -1), (230, -1), (240, 130)])   # whole windows; a cut last window; updates stop early
def test_ar_video_interleaved(use_momentum, weight_norm, use_moun, repeat, L, update_length):
    say("ar video", use_momentum, weight_norm, use_moun, repeat, L, update_length)
    b, d, dh, mb = 2, 64, 128, 40
    inp = problem(b, L, d, dh, 14, torch.bfloat16, momentum=use_momentum)

    def hip(t):
        r = ar_video.ar_fast_weight_swish_glu_weight_norm_mini_batch_with_momentum(
            *args9(t), 0.5, repeat, mb, update_length, 2 * mb, use_moun, 3, weight_norm, t["momentum"], use_momentum)
        assert len(r) == 4
        return r[0]

    def orc(t, num):
        return O.ar_fast_weight_swish_glu_weight_norm_mini_batch(
            *args9(t), 0.5, repeat, mb, update_length, 2 * mb, use_moun, 3, weight_norm, t["momentum"], use_momentum, num=num)[0]
    if use_moun:
        res, ref, r64, floors = run_both(hip, orc, inp, AC, ref64=True, floor=True)
        assert_within_order_floor(res, ref, floors, "ar-video", r64)
    else:
        res, ref = run_both(hip, orc, inp, AC)
        errs = compare(res, ref)
        say("  ", errs)
        assert max(errs.values()) < 1e-2


@pytest.mark.parametrize("act,d,dh,L,mb", [(torch.float32, 64, 64, 96, 64), (torch.bfloat16, 128, 128, 200, 128),
                                           (torch.bfloat16, 384, 384, 300, 256)])
def test_ar_video_inference_repeat_accumulates_kv_grads(act, d, dh, L, mb):
    """num_repeat > 1 re-uses the same k, v rows in several updates: their gradients must accumulate (in bf16 the
    second touch happens inside the launch that also holds the token reduction)."""
    say("ar video inference, num_repeat=2", act, d, dh, L, mb)
    b = 2
    inp = problem(b, L, d, dh, 15, act, momentum=False, lr_shift=-1.0)
    hip = lambda t: ar_video.ar_fast_weight_swish_glu_weight_norm_mini_batch_inference(
        *args9(t), 1.0, 2, mb, True, False, 3, True)[0]
    orc = lambda t, num: O.ar_fast_weight_swish_glu_weight_norm_mini_batch_inference(
        *args9(t), 1.0, 2, mb, True, False, 3, True, num=num)[0]
    res, ref = run_both(hip, orc, inp, PLAIN if act == torch.float32 else AC)
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < (1e-4 if act == torch.float32 else 1e-2)


INF_M = ar_video.ar_fast_weight_swish_glu_weight_norm_mini_batch_inference_with_momentum
INF_M_ORACLE = O.ar_fast_weight_swish_glu_weight_norm_mini_batch_inference_with_momentum


@pytest.mark.parametrize("d,dh,act,use_moun,weight_norm,repeat", [
    (64, 128, torch.float32, False, True, 1), (64, 128, torch.float32, False, False, 2),
    (128, 128, torch.float32, True, True, 1),       # fp32 Newton-Schulz against float64 (exact arithmetic)
    (64, 128, torch.bfloat16, False, True, 2), (128, 128, torch.bfloat16, True, True, 1),
    (384, 384, torch.bfloat16, True, True, 2),      # fused Newton-Schulz, momentum step in the reduction's epilogue
    (40, 136, torch.bfloat16, False, True, 1)])
def test_ar_video_inference_with_carried_momentum_state(d, dh, act, use_moun, weight_norm, repeat):
    """ar_lact_swa_repeat_sp.py:197-339: the first update continues from the states of an earlier call."""
    say("ar video inference with momentum state", d, dh, act, use_moun, weight_norm, repeat)
    b, L, mb = 3, 200, 128
    inp = problem(b, L, d, dh, 21, act, momentum=True, lr_shift=-1.0)
    gen = torch.Generator().manual_seed(77)
    M = [0.02 * torch.randn(w.shape, generator=gen) for w in (inp["w0"], inp["w1"], inp["w2"])]
    exact = use_moun and act == torch.float32
    num = EXACT if exact else (AC if act == torch.bfloat16 else PLAIN)
    cast = (lambda t: t.double()) if exact else (lambda t: t)
    c = {n: (None if t is None else cast(t)) for n, t in inp.items()}
    with torch.no_grad():
        ref = INF_M_ORACLE(*args9(c), 0.5, repeat, mb, True, use_moun, 3, weight_norm, c["momentum"],
                           cast(M[0]), cast(M[1]), cast(M[2]), True, num=num)
        g = clone_to(inp, DEV, grad=False)
        Mg = [m.to(DEV) for m in M]
        run = lambda: INF_M(*args9(g), 0.5, repeat, mb, True, use_moun, 3, weight_norm, g["momentum"], Mg[0], Mg[1],
                            Mg[2], True)
        if exact:
            with ops.newton_schulz_mode(ops.NS_FP32):
                res = run()
        else:
            res = run()
        torch.cuda.synchronize()
        names = ["out", "w0", "w1", "w2", "m0", "m1", "m2"]
        errs = {n: O.rel_l2(r, f) for n, r, f in zip(names, res, ref)}
        say("  ", errs)
        if use_moun and not exact:
            # bf16 Newton-Schulz: bounded by the order-only floor
            floors = {n: 0.0 for n in names}
            for v in O.order_variants(num):
                var = INF_M_ORACLE(*args9(c), 0.5, repeat, mb, True, use_moun, 3, weight_norm, c["momentum"],
                                   M[0], M[1], M[2], True, num=v)
                for n, x, f in zip(names, var, ref):
                    floors[n] = max(floors[n], O.rel_l2(x, f))
            say("   floors", floors)
            for n in names:
                assert errs[n] <= 1.5 * floors[n] + 1e-3, n
        else:
            tol = 1e-3 if exact else (1e-2 if act == torch.bfloat16 else 1e-4)
            assert max(errs.values()) < tol
        # without a state the same call differs (the state is really used)
        bare = INF_M(*args9(g), 0.5, repeat, mb, True, use_moun, 3, weight_norm, g["momentum"], None, None, None, True)
        assert O.rel_l2(bare[4], res[4]) > 1e-2


def test_carried_momentum_state_equals_one_longer_program_bitwise():
    """Two calls that hand weights and states over do the arithmetic of one call with two updates (no weight norm,
    so nothing is re-derived from the handed-over weights): same kernels, same bits."""
    say("carried state: two calls against one")
    inp = problem(2, 160, 64, 128, 22, torch.float32, momentum=True, lr_shift=-1.0)
    with torch.no_grad():
        g = clone_to(inp, DEV, grad=False)
        both = INF_M(*args9(g), 0.7, 2, 96, True, False, 3, False, g["momentum"], None, None, None, True)
        one = INF_M(*args9(g), 0.7, 1, 96, True, False, 3, False, g["momentum"], None, None, None, True)
        two = INF_M(one[1], one[2], one[3], g["q"], g["k"], g["v"], g["lr0"], g["lr1"], g["lr2"], 0.7, 1, 96, True, False,
                    3, False, g["momentum"], one[4], one[5], one[6], True)
        torch.cuda.synchronize()
        for n, a, b_ in zip(["out", "w0", "w1", "w2", "m0", "m1", "m2"], both, two):
            assert torch.equal(a, b_), n
        # no update: states and weights pass through, momentum off: states handed back as given
        idle = INF_M(*args9(g), 0.7, 1, 96, False, False, 3, True, g["momentum"], one[4], one[5], one[6], True)
        assert idle[4] is one[4] and torch.equal(idle[1], g["w0"])
        off = INF_M(*args9(g), 0.7, 1, 96, True, False, 3, True, None, None, None, None, False)
        assert off[4] is None
    # a carried state has no backward pass: refused when a gradient is wanted
    gg = clone_to(inp, DEV)
    with pytest.raises(RuntimeError, match="inference"):
        INF_M(*args9(gg), 0.7, 1, 96, True, False, 3, True, gg["momentum"], one[4], one[5], one[6], True)


def test_fast_weight_inference_cache_follows_the_layer_protocol():
    """ar_lact_swa_repeat_sp.py:998-1053,1147-1148: conditional and guidance sequences alternate, each with its own
    weights and momentum states; both restart from the layer's parameters until each has been updated once."""
    say("fast-weight inference cache")
    b, L, d, dh = 2, 96, 64, 64
    base = problem(b, L, d, dh, 23, torch.float32, momentum=True, lr_shift=-1.0)
    chunks = [problem(b, L, d, dh, 30 + i, torch.float32, momentum=True, lr_shift=-1.0) for i in range(6)]
    do_update = [True, True, False, False, True, True]
    cache = ar_video.FastWeightInferenceCache(use_momentum=True)
    held = {False: None, True: None}      # the oracle's copy of the protocol, written out call by call
    cfg = False
    with torch.no_grad():
        W = [base[n].to(DEV) for n in ("w0", "w1", "w2")]
        for i, (ch, upd) in enumerate(zip(chunks, do_update)):
            g = clone_to(ch, DEV, grad=False)
            out = cache.step(W[0], W[1], W[2], g["q"], g["k"], g["v"], g["lr0"], g["lr1"], g["lr2"], 0.5, do_update=upd,
                             frames=3, fw_momentum=g["momentum"], mini_batch_size=64)
            fresh = held[False] is None or held[True] is None
            st = (base["w0"], base["w1"], base["w2"], None, None, None) if fresh else held[cfg]
            ref = INF_M_ORACLE(st[0], st[1], st[2], ch["q"], ch["k"], ch["v"], ch["lr0"], ch["lr1"], ch["lr2"], 0.5, 1, 64,
                               upd, False, 3, True, ch["momentum"], st[3], st[4], st[5], True, num=PLAIN)
            if upd:
                held[cfg] = tuple(ref[1:])
            cfg = not cfg
            e = O.rel_l2(out, ref[0])
            say("   call", i, "update" if upd else "apply", "err", e)
            assert e < 1e-4
    assert cache.frame_offset == 6 and cache.cfg_seq is False      # two updating conditional calls, three frames each
    cache.reset()
    assert cache.cur is None and cache.frame_offset == 0


def test_video_model_shape_full_size_equals_its_inference_rollout():
    """The video model's own shape (lact_ar_chunk3f_1.3B.yaml: 2 heads of 768, hidden 1536, 4680-token windows,
    update_every 9360, 7 windows = 60840 tokens, no Muon), too large for the CPU oracle: the training-time program
    must equal the step-by-step inference rollout (apply on the first window; then update on each clean window and
    apply on it and the noisy window that follows, weights handed from call to call) -- both paths are checked
    against the oracle at small sizes above.  bf16 bound 1e-2; gradients finite and linear in the upstream."""
    b, d, dh, mb, ue = 2, 768, 1536, 4680, 9360
    L = mb + 6 * ue
    say("video model shape, full size", b, d, dh, L)
    inp = O.make_inputs(b, L, d, dh, seed=5, act_dtype=torch.bfloat16, distinct_heads=2)
    g = clone_to(inp, DEV)
    go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(3)).bfloat16().to(DEV)
    names = [n for n in NAMES if g.get(n) is not None and n != "momentum"]

    def run(upstream):
        res = ar_video.ar_fast_weight_swish_glu_weight_norm_mini_batch(*args9(g), 1.0, 1, mb, -1, ue, False, 5, True)
        return res, torch.autograd.grad(res[0], [g[n] for n in names], upstream)
    res, g1 = run(go)
    _, g2 = run(go * 2)
    for n, a, c in zip(names, g1, g2):
        assert torch.isfinite(a.float()).all(), n
        assert O.rel_l2(c.float().cpu(), 2 * a.float().cpu()) < 5e-3, n
    inf = ar_video.ar_fast_weight_swish_glu_weight_norm_mini_batch_inference
    with torch.no_grad():
        w = [g["w0"], g["w1"], g["w2"]]
        sl = lambda t, a, e: t[:, a:e]
        outs = [inf(*w, sl(g["q"], 0, mb), sl(g["k"], 0, mb), sl(g["v"], 0, mb), sl(g["lr0"], 0, mb), sl(g["lr1"], 0, mb),
                    sl(g["lr2"], 0, mb), 1.0, 1, mb, False, False, 5, True)[0]]
        for s0 in range(mb, L, ue):
            r = inf(*w, sl(g["q"], s0, s0 + ue), sl(g["k"], s0, s0 + mb), sl(g["v"], s0, s0 + mb), sl(g["lr0"], s0, s0 + mb),
                    sl(g["lr1"], s0, s0 + mb), sl(g["lr2"], s0, s0 + mb), 1.0, 1, mb, True, False, 5, True)
            outs.append(r[0])
            w = list(r[1:4])
        e_out = O.rel_l2(torch.cat(outs, 1).cpu(), res[0].detach().cpu())
        e_w = max(O.rel_l2(a.cpu(), c.detach().cpu()) for a, c in zip(w, res[1:4]))
    say("   rollout vs program: out", e_out, "final weights", e_w)
    assert e_out < 1e-2 and e_w < 2e-3


def test_fused_newton_schulz_barrier_timeout_ends_every_kernel_and_poisons_the_step():
    """The blocks of the fused Newton-Schulz kernel wait for each other with a bounded poll.  The host forces the
    bound to one poll: blocks give up at (nearly) every barrier, read partner tiles too early, raise the error word
    -- and still run to their end.  The step's results must be NaN (never silently wrong numbers), and the next
    call with the default bound must be right again."""
    from lact_amd import _lib
    say("fused Newton-Schulz: forced barrier timeout")
    inp = problem(4, 3 * 128, 256, 256, 41, torch.bfloat16, momentum=True, lr_shift=-1.0)   # 4 or 8 blocks per matrix
    hip, _ = block_causal_pair(128, True)

    def run():
        g = clone_to(inp, DEV)
        out = hip(g)
        go = torch.randn(out.shape, generator=torch.Generator().manual_seed(3)).bfloat16().to(DEV)
        grads = grads_of(out, g, go)
        torch.cuda.synchronize()
        return out.detach().float().cpu(), {n: v.detach().float().cpu() for n, v in grads.items()}
    good_out, good = run()
    assert torch.isfinite(good_out).all()
    L = _lib.lib()
    assert L.lact_check_async_error() == 0                     # nothing timed out so far in this process
    prev = L.lact_set_option(_lib.OPT_NS_BARRIER_SPIN_LIMIT, 1)
    try:
        assert prev > 1
        bad_out, bad = run()
    finally:
        assert L.lact_set_option(_lib.OPT_NS_BARRIER_SPIN_LIMIT, 0) == 1
    # the time-outs reach the host: a count and a message, once
    with pytest.raises(RuntimeError, match="timed out"):
        ops.check_async_error()
    assert L.lact_check_async_error() == 0
    # ... and the fused kernel is off from then on (whatever held the compute units may still be there): the caller
    # switches it back on
    assert L.lact_set_option(_lib.OPT_FUSED_NEWTON_SCHULZ, 1) == 0
    assert torch.equal(bad_out[:, :128], good_out[:, :128])      # first chunk: initial weights, no Newton-Schulz yet
    assert torch.isnan(bad_out[:, 128:]).all()                   # everything behind the first update
    assert torch.isnan(bad["w0"]).all() and torch.isnan(bad["k"][:, :128]).all()
    again_out, again = run()
    assert torch.equal(again_out, good_out) and all(torch.equal(again[n], good[n]) for n in good)


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_output_rows_written_twice_belong_to_the_later_apply(act):
    """A program may write an output row in several apply steps; the reference's slice assignment lets the last
    write win and autograd sends the overwritten values no gradient.  Here: rows 48..112 are written by the first
    apply (initial weights) and again by the second (updated weights), rows 112..160 only by the second, and a
    third apply rewrites 0..16 -- forward and every gradient against the oracle."""
    say("overwritten output rows", act)
    b, L, d, dh = 2, 160, 64, 128
    inp = problem(b, L, d, dh, 52, act, momentum=True, lr_shift=-1.0)
    prog_steps = ((LACT_APPLY, 0, 112, 0), (ops.LACT_UPDATE, 0, 64, 0), (LACT_APPLY, 48, 160, 48),
                  (ops.LACT_UPDATE, 64, 128, 0), (LACT_APPLY, 0, 16, 0))
    prog = ops.Program(steps=prog_steps, out_len=L)
    hip = lambda t: ops.run_program(prog, *args9(t), t["momentum"])[0]
    osteps = [O.Step(O.APPLY if k == LACT_APPLY else O.UPDATE, s0, e0) for k, s0, e0, _ in prog_steps]
    orc = lambda t, num: O.run_program(*args9(t), osteps, num=num, momentum=t["momentum"])[0]
    res, ref = run_both(hip, orc, inp, PLAIN if act == torch.float32 else AC)
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < (1e-4 if act == torch.float32 else 1e-2)


def test_program_with_more_than_256_updates():
    """Per-update quantities that are written by one launch for the whole program (momentum means, momentum and
    learning-rate gradients) go in batches of 256 updates: 300 chunks of 64 tokens, fp32 against the oracle."""
    say("300 updates")
    b, d, dh, C = 1, 64, 64, 64
    L = 300 * C + 20
    inp = problem(b, L, d, dh, 61, torch.float32, momentum=True, lr_shift=-4.0)
    res, ref = run_both(*block_causal_pair(C, False), inp, PLAIN)
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < 1e-4


def _random_program(rng, L):
    """2 to 7 steps with arbitrary (also overlapping, also repeated) token ranges; at least one apply at the end."""
    steps = []
    for _ in range(int(rng.integers(2, 8))):
        a = int(rng.integers(0, L - 8))
        e = int(rng.integers(a + 4, min(L, a + 200) + 1))
        kind = LACT_APPLY if rng.random() < 0.45 else ops.LACT_UPDATE
        steps.append((kind, a, e, a if kind == LACT_APPLY else 0))
    a = int(rng.integers(0, L // 2))
    steps.append((LACT_APPLY, a, L, a))
    return tuple(steps)


@pytest.mark.parametrize("seed", list(range(20)))
def test_random_programs_match_oracle(seed):
    """Differential test over random valid programs (random shapes, step lists with overlapping and repeated ranges,
    momentum / pre-norm / weight-norm / Muon switches): forward and every gradient against the oracle.  fp32
    activations; Newton-Schulz in fp32 against float64 arithmetic (1e-3), everything else at the fp32 bound 1e-4."""
    rng = np.random.default_rng(1000 + seed)
    b = int(rng.integers(1, 3))
    d = int(rng.choice([16, 40, 64, 128]))
    dh = int(rng.choice([24, 64, 128, 192]))
    L = int(rng.integers(60, 400))
    momentum, prenorm, weight_norm = bool(rng.random() < 0.6), bool(rng.random() < 0.3), bool(rng.random() < 0.8)
    muon = bool(rng.random() < 0.4)
    steps = _random_program(rng, L)
    say("random program", seed, dict(b=b, d=d, dh=dh, L=L, momentum=momentum, prenorm=prenorm, weight_norm=weight_norm, muon=muon), steps)
    inp = problem(b, L, d, dh, 2000 + seed, torch.float32, momentum=momentum, lr_shift=-2.0)
    coeffs = O.ns_coeff_table("llm", 5) if muon else None
    prog = ops.Program(steps=steps, out_len=L, ns_coeffs=coeffs, prenorm=prenorm, weight_norm=weight_norm, ns_mode=ops.NS_FP32)
    osteps = [O.Step(O.APPLY if k == LACT_APPLY else O.UPDATE, s0, e0) for k, s0, e0, _ in steps]

    def hip(t):
        return ops.run_program(prog, *args9(t), t["momentum"])[0]

    def orc(t, num):
        return O.run_program(*args9(t), osteps, num=num, ns_coeffs=coeffs, momentum=t["momentum"], prenorm=prenorm,
                             weight_norm=weight_norm)[0]
    g = clone_to(inp, DEV)
    out = hip(g)
    go = torch.randn(out.shape, generator=torch.Generator().manual_seed(3))
    res = {"out": out, **grads_of(out, g, go.to(DEV))}
    torch.cuda.synchronize()
    if muon:
        c = clone_to(inp, "cpu", dtype_map=lambda t: torch.float64)
        o = orc(c, EXACT)
        ref = {"out": o, **grads_of(o, c, go.double())}
        tol = 1e-3
    else:
        c = clone_to(inp, "cpu")
        o = orc(c, PLAIN)
        ref = {"out": o, **grads_of(o, c, go)}
        tol = 1e-4
    errs = compare(res, ref)
    say("  ", {n: float("%.2e" % e) for n, e in errs.items()})
    assert max(errs.values()) < tol


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_programs_match_oracle_bf16(seed):
    """The same differential test on the bf16 path (asynchronous-copy kernels: d, dh multiples of 64; longer
    ranges), Muon off so that the north-star bound 1e-2 applies outright; the momentum gradient (one dot product per
    head and chunk) is held to the oracle's own distance from float64 where that distance is large."""
    rng = np.random.default_rng(5000 + seed)
    b = int(rng.integers(1, 4))
    d = int(rng.choice([64, 128, 192]))
    dh = int(rng.choice([64, 128, 256]))
    L = int(rng.integers(200, 900))
    momentum, prenorm, weight_norm = bool(rng.random() < 0.6), bool(rng.random() < 0.3), bool(rng.random() < 0.8)
    steps = []
    for _ in range(int(rng.integers(2, 7))):
        a = int(rng.integers(0, L - 70))
        e = int(rng.integers(a + 64, min(L, a + 600) + 1))
        kind = LACT_APPLY if rng.random() < 0.45 else ops.LACT_UPDATE
        steps.append((kind, a, e, a if kind == LACT_APPLY else 0))
    a = int(rng.integers(0, L // 2))
    steps.append((LACT_APPLY, a, L, a))
    steps = tuple(steps)
    say("random bf16 program", seed, dict(b=b, d=d, dh=dh, L=L, momentum=momentum, prenorm=prenorm, weight_norm=weight_norm), steps)
    inp = problem(b, L, d, dh, 6000 + seed, torch.bfloat16, momentum=momentum, lr_shift=-3.0)
    prog = ops.Program(steps=steps, out_len=L, prenorm=prenorm, weight_norm=weight_norm)
    osteps = [O.Step(O.APPLY if k == LACT_APPLY else O.UPDATE, s0, e0) for k, s0, e0, _ in steps]
    hip = lambda t: ops.run_program(prog, *args9(t), t["momentum"])[0]
    orc = lambda t, num: O.run_program(*args9(t), osteps, num=num, momentum=t["momentum"], prenorm=prenorm, weight_norm=weight_norm)[0]
    res, ref = run_both(hip, orc, inp, AC)
    errs = compare(res, ref)
    say("  ", {n: float("%.2e" % e) for n, e in errs.items()})
    for n, e in errs.items():
        assert e < 1e-2, n


# ---- size-independent properties at the benchmark size ----------------------------------------------
def full_size_properties(b, L, d, dh, C, seed, single_update):
    inp = O.make_inputs(b, L, d, dh, seed=seed, act_dtype=torch.bfloat16, distinct_heads=4)
    g = clone_to(inp, DEV)
    go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(3)).bfloat16().to(DEV)
    last = ((L - 1) // C) * C        # first row of the last chunk

    def run(t, upstream=None):
        out = T.block_causal_lact_swiglu(*args9(t), C, True, t["momentum"])
        return out, grads_of(out, t, go if upstream is None else upstream)
    out1, gr1 = run(g)
    out2, gr2 = run(g)
    assert torch.equal(out1, out2) and all(torch.equal(gr1[n], gr2[n]) for n in gr1)      # deterministic
    assert all(torch.isfinite(v.float()).all() for v in gr1.values()) and torch.isfinite(out1.float()).all()
    ref0 = O.swiglu_apply(inp["w0"], inp["w1"], inp["w2"], inp["q"][:, :C], AC)
    assert O.rel_l2(out1[:, :C], ref0) < 1e-3
    # causality: k, v of the last chunk are never read; their gradients are exactly zero
    assert float(gr1["k"][:, last:].abs().max()) == 0.0 and float(gr1["v"][:, last:].abs().max()) == 0.0
    assert float(gr1["lr0"][:, last:].abs().max()) == 0.0 and float(gr1["momentum"][:, last:].abs().max()) == 0.0
    t2 = clone_to(inp, DEV)
    with torch.no_grad():
        t2["k"][:, last + 5] += 1.0
        t2["v"][:, last + 7] -= 1.0
        t2["q"][:, last + 9] += 1.0                                    # only row last+9 of the output may move
    out3, _ = run(t2)
    keep = torch.ones(L, dtype=torch.bool); keep[last + 9] = False
    assert torch.equal(out3[:, keep.to(DEV)], out1[:, keep.to(DEV)])
    assert not torch.equal(out3[:, last + 9], out1[:, last + 9])
    # heads never interact: a permutation of the batch permutes outputs and gradients bit-exactly
    perm = torch.randperm(b, generator=torch.Generator().manual_seed(1)).to(DEV)
    t3 = {n: (None if v is None else v.detach()[perm].clone().requires_grad_(True)) for n, v in g.items()}
    out4, gr4 = run(t3, go[perm])
    assert torch.equal(out4, out1[perm]) and torch.equal(gr4["w1"], gr1["w1"][perm]) and torch.equal(gr4["k"], gr1["k"][perm])
    if single_update:
        # nothing is carried into the only update: d loss / d momentum is <g, M_prev> = 0
        assert float(gr1["momentum"].abs().max()) == 0.0
    else:
        # the first chunk's momentum weighs no earlier state; later chunks' momentum does
        assert float(gr1["momentum"][:, :C].abs().max()) == 0.0 and float(gr1["momentum"][:, C:last].abs().max()) > 0.0


@pytest.mark.parametrize("cfg,b,L,d,dh,C,seed", [
    (1, 16, 4096, 384, 384, 2048, 1001),          # config 1 whole: one update, two applies
    (2, 4, 3 * 2048, 384, 384, 2048, 1002),       # config 2, first three chunks: two chained updates with momentum carry
    (4, 12, 3 * 4680, 128, 256, 4680, 1004)])     # config 4, first three chunks (73 x 64 + 8 tokens each)
def test_config_full_size_against_oracle(cfg, b, L, d, dh, C, seed):
    """The benchmark shapes at their full b, d, dh and chunk size (Muon, momentum 0.9, bf16, forward + backward):
    output and all ten gradients against the oracle, bounded by the order-only floor measured on the same inputs."""
    say("config", cfg, "full size against the oracle", b, L, d, dh, C)
    inp = O.make_inputs(b, L, d, dh, seed=seed, act_dtype=torch.bfloat16, distinct_heads=4)
    res, ref, floors = run_both(*block_causal_pair(C, True), inp, AC, floor=True)
    if cfg == 1:
        # nothing is carried into the only update: d loss / d momentum is exactly zero on both sides
        assert float(res["momentum"].abs().max()) == 0.0 and float(ref["momentum"].abs().max()) == 0.0
    assert_within_order_floor(res, ref, floors, f"config-{cfg}")
    if cfg == 1:
        # The momentum state after a single update is the PRE-Muon gradient dw (ttt_operation.py:170-179): Newton-Schulz
        # never touches it, so nothing amplifies and it is held to 1e-3, far below the floor of the output.
        steps = ops.block_causal_steps(L, C)
        prog = ops.Program(steps=steps, out_len=L, ns_coeffs=O.NS5_COEFFS)
        g = clone_to(inp, DEV, grad=False)
        with torch.no_grad():
            _, _, ms = ops.run_program(prog, *args9(g), g["momentum"])
        osteps = [O.Step(O.APPLY if k == LACT_APPLY else O.UPDATE, s, e) for k, s, e, _ in steps]
        with torch.no_grad():
            _, _, mref = O.run_program(*args9(inp), osteps, num=AC, ns_coeffs=O.NS5_COEFFS, momentum=inp["momentum"])
        for j, (a, r) in enumerate(zip(ms, mref)):
            e = O.rel_l2(a, r)
            say(f"   config-1 momentum state {j}: hip-vs-oracle {e:.2e}")
            assert e <= 1e-3, (j, e)


def test_config1_full_size_properties():
    """BASELINE config 1 (b=16, L=4096, d=dh=384, chunk 2048, Muon, momentum 0.9, fwd+bwd) at full size:
    determinism, block causality, head independence -- bit-exact checks no oracle run is needed for --
    plus the first chunk against the oracle (its output does not depend on any update)."""
    say("config 1 full-size properties")
    full_size_properties(16, 4096, 384, 384, 2048, 1001, True)


def test_config2_full_size_properties():
    """BASELINE config 2 (b=4, L=32768, d=dh=384, chunk 2048: 15 chained updates) at full size."""
    say("config 2 full-size properties")
    full_size_properties(4, 32768, 384, 384, 2048, 1002, False)


def test_config4_full_size_properties():
    """BASELINE config 4 (b=12, L=32760, d=128, dh=256, chunk 4680 = 73 x 64 + 8 tokens: ragged token tiles) at
    full size."""
    say("config 4 full-size properties")
    full_size_properties(12, 32760, 128, 256, 4680, 1004, False)


def test_forward_only_and_output_only_calls():
    """Under torch.no_grad the descriptor is forward-only (nothing kept for a backward) and the output has the same
    bits as in a training call; a program with return_state=False returns None for the final weights and momentum
    states, with the same output."""
    say("forward-only / output-only")
    b, L, d, dh, C = 2, 3 * 128 + 9, 128, 128, 128
    inp = problem(b, L, d, dh, seed=31, act=torch.bfloat16)
    t = clone_to(inp, DEV)
    out_train = T.block_causal_lact_swiglu(*args9(t), C, True, t["momentum"])
    with torch.no_grad():
        out_infer = T.block_causal_lact_swiglu(*args9(t), C, True, t["momentum"])
    assert torch.equal(out_train, out_infer) and not out_infer.requires_grad
    steps = ops.block_causal_steps(L, C)
    full = ops.Program(steps=steps, out_len=L, ns_coeffs=ops.NS5_COEFFS)
    lean = ops.Program(steps=steps, out_len=L, ns_coeffs=ops.NS5_COEFFS, return_state=False)
    o1, w1, m1 = ops.run_program(full, *args9(t), t["momentum"])
    o2, w2, m2 = ops.run_program(lean, *args9(t), t["momentum"])
    assert torch.equal(o1, o2) and torch.equal(o1, out_train)
    assert all(w is not None for w in w1) and all(m is not None for m in m1)
    assert all(w is None for w in w2) and all(m is None for m in m2)
    g1 = grads_of(o1, t, torch.ones_like(o1))
    g2 = grads_of(o2, t, torch.ones_like(o2))
    assert all(torch.equal(g1[n], g2[n]) for n in g1)


def test_graph_capture_replays_match_eager():
    """Forward + backward captured into a HIP graph (the library forks and joins its side streams with events
    only, and clears memory with kernels): three replays on fresh inputs, with eager work and synchronisations in
    between, each bit-identical to the eager call on the same inputs."""
    say("graph capture")
    b, L, d, dh, C = 2, 3 * 384, 384, 384, 384
    inp = problem(b, L, d, dh, seed=55, act=torch.bfloat16)
    st = clone_to(inp, DEV)
    go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(9)).bfloat16().to(DEV)

    def run():
        out = T.block_causal_lact_swiglu(*args9(st), C, True, st["momentum"])
        return out, grads_of(out, st, go)
    run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):               # warm-up on a side stream, as torch asks before a capture
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g, grads_g = run()
    torch.cuda.synchronize()
    gen = torch.Generator().manual_seed(123)
    for rep in range(3):
        with torch.no_grad():
            st["q"].copy_(torch.nn.functional.normalize(torch.randn(b, L, d, generator=gen), dim=-1).bfloat16())
            st["v"].copy_(torch.randn(b, L, d, generator=gen).bfloat16())
            st["lr1"].copy_(torch.nn.functional.softplus(torch.randn(b, L, 1, generator=gen) - 3.0))
        graph.replay()
        torch.cuda.synchronize()
        out_r, grads_r = out_g.clone(), {n: g.clone() for n, g in grads_g.items()}
        out_e, grads_e = run()
        torch.cuda.synchronize()
        assert torch.equal(out_r, out_e), rep
        for n in grads_e:
            assert torch.equal(grads_r[n], grads_e[n]), (rep, n)


def test_calls_on_two_caller_streams():
    """Two independent problems enqueued on two caller streams at once (forward and backward each), as a caller with
    its own stream pool would: the library's side streams, the ordering of the fused Newton-Schulz kernels across
    streams and the shared event pool must not mix them up.  Same bits as the same calls on one stream."""
    say("two caller streams")
    b, L, d, dh, C = 2, 3 * 384, 384, 384, 384
    inps = [problem(b, L, d, dh, seed=91 + i, act=torch.bfloat16) for i in range(2)]
    gos = [torch.randn(b, L, d, generator=torch.Generator().manual_seed(7 + i)).bfloat16().to(DEV) for i in range(2)]

    def run(streams):
        ts = [clone_to(inp, DEV) for inp in inps]
        torch.cuda.synchronize()
        outs, grads = [None, None], [None, None]
        for rep in range(2):
            for i in range(2):
                with torch.cuda.stream(streams[i]):
                    outs[i] = T.block_causal_lact_swiglu(*args9(ts[i]), C, True, ts[i]["momentum"])
            for i in range(2):
                with torch.cuda.stream(streams[i]):
                    grads[i] = grads_of(outs[i], ts[i], gos[i])
        torch.cuda.synchronize()
        return outs, grads
    cur = torch.cuda.current_stream()
    o1, g1 = run([cur, cur])
    o2, g2 = run([torch.cuda.Stream(), torch.cuda.Stream()])
    for i in range(2):
        assert torch.equal(o1[i], o2[i])
        for n in g1[i]:
            assert torch.equal(g1[i][n], g2[i][n]), n


def test_calls_from_two_host_threads():
    """Two host threads, each with a stream of its own, run forward + backward of different problems at the same
    time (the enqueue of a program is serialised inside the library; execution is not).  Same bits as one thread."""
    say("two host threads")
    import threading
    b, L, d, dh, C = 2, 3 * 256, 128, 256, 256
    inps = [problem(b, L, d, dh, seed=191 + i, act=torch.bfloat16) for i in range(2)]
    gos = [torch.randn(b, L, d, generator=torch.Generator().manual_seed(17 + i)).bfloat16().to(DEV) for i in range(2)]

    def one(i, stream, res):
        try:
            with torch.cuda.stream(stream):
                for _ in range(3):
                    t = clone_to(inps[i], DEV)
                    out = T.block_causal_lact_swiglu(*args9(t), C, True, t["momentum"])
                    res[i] = (out, grads_of(out, t, gos[i]))
            stream.synchronize()
        except Exception as e:   # surfaces in the main thread below
            res[i] = e
    ref = [None, None]
    for i in range(2):
        one(i, torch.cuda.current_stream(), ref)
    torch.cuda.synchronize()
    res = [None, None]
    th = [threading.Thread(target=one, args=(i, torch.cuda.Stream(), res)) for i in range(2)]
    for t_ in th:
        t_.start()
    for t_ in th:
        t_.join()
    torch.cuda.synchronize()
    for i in range(2):
        assert not isinstance(res[i], Exception), res[i]
        assert torch.equal(res[i][0], ref[i][0])
        for n in ref[i][1]:
            assert torch.equal(res[i][1][n], ref[i][1][n]), n


@pytest.mark.parametrize("prenorm", [False, True])
def test_stream_overlap_is_bit_identical(prenorm):
    """The apply steps run on the library's second stream beside the update chain (forked and joined with
    events).  With the overlap switched off everything is enqueued on the caller's stream: both must give the
    same bits, over several chunks (the apply steps' weight-gradient buffers alternate by weight version)
    and over back-to-back calls."""
    say("stream overlap on/off, prenorm", prenorm)
    from lact_amd import _lib
    b, L, d, dh, C = 4, 5 * 256, 128, 128, 256
    inp = problem(b, L, d, dh, seed=77, act=torch.bfloat16)
    go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(5)).bfloat16().to(DEV)
    fn = T.prenorm_block_causal_lact_swiglu if prenorm else T.block_causal_lact_swiglu

    def run():
        res = []
        for _ in range(3):                       # back-to-back: the second stream's work of one call meets the next
            t = clone_to(inp, DEV)
            out = fn(*args9(t), C, True, t["momentum"])
            res.append((out, grads_of(out, t, go)))
        torch.cuda.synchronize()
        return res
    L_ = _lib.lib()
    prev = L_.lact_set_option(_lib.OPT_STREAM_OVERLAP, 1)
    try:
        on = run()
        L_.lact_set_option(_lib.OPT_STREAM_OVERLAP, 0)
        off = run()
    finally:
        L_.lact_set_option(_lib.OPT_STREAM_OVERLAP, prev)
    for (o1, g1), (o0, g0) in zip(on, off):
        assert torch.equal(o1, o0)
        for n in g0:
            assert torch.equal(g1[n], g0[n]), n
    assert torch.equal(on[0][0], on[2][0]) and all(torch.equal(on[0][1][n], on[2][1][n]) for n in on[0][1])


@pytest.mark.parametrize("b,L,d,dh,C,muon", [
    (2, 3 * 128 + 40, 128, 128, 128, False),      # ragged last token tile, one hidden tile
    (3, 2 * 300 + 50, 64, 192, 300, True),        # dh = 128 + 64: a half-valid hidden tile; chunk not a multiple of 128
    (5, 3 * 256, 128, 256, 256, True),            # batch not a multiple of 8 (tile map by rows of tiles)
    (16, 2 * 1024 + 7, 384, 384, 1024, True),     # config-1 head shape, several tiles per block
    (1, 2 * 64, 64, 64, 64, False)])              # fewer tiles than compute units, one K-step per phase
def test_persistent_tiles_are_bit_identical(b, L, d, dh, C, muon):
    """The hidden-stage kernels as persistent blocks (copy waves running ahead across tiles while the matrix waves run
    the previous tile's epilogue) against one tile per block: the same arithmetic in the same order, so the same bits
    in the output and in every gradient."""
    say("persistent tiles on/off", b, L, d, dh, C, muon)
    from lact_amd import _lib
    inp = problem(b, L, d, dh, seed=55, act=torch.bfloat16)
    go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(8)).bfloat16().to(DEV)

    def run():
        res = []
        for _ in range(2):
            t = clone_to(inp, DEV)
            out = T.block_causal_lact_swiglu(*args9(t), C, muon, t["momentum"])
            res.append((out, grads_of(out, t, go)))
        torch.cuda.synchronize()
        return res
    L_ = _lib.lib()
    prev = L_.lact_set_option(_lib.OPT_PERSISTENT_TILES, 7)      # all three hidden-stage kernels persistent
    try:
        on = run()
        L_.lact_set_option(_lib.OPT_PERSISTENT_TILES, 0)
        off = run()
    finally:
        L_.lact_set_option(_lib.OPT_PERSISTENT_TILES, prev)
    for (o1, g1), (o0, g0) in zip(on, off):
        assert torch.isfinite(o1.float()).all()
        assert torch.equal(o1, o0)
        for n in g0:
            assert torch.equal(g1[n], g0[n]), (n, O.rel_l2(g1[n], g0[n]))
    assert all(torch.equal(on[0][1][n], on[1][1][n]) for n in on[0][1])


@pytest.mark.parametrize("b,L,d,dh,C,muon", [
    (3, 3 * 256 + 40, 128, 256, 256, True),       # the shape class where the library recomputes by itself (d <= 128)
    (2, 2 * 1024 + 7, 384, 384, 1024, True),      # ... and where it keeps
    (2, 3 * 128, 64, 192, 128, False)])
def test_kept_and_recomputed_update_backward_agree(b, L, d, dh, C, muon):
    """The update's backward from the pre-activations the forward kept against the backward that recomputes them
    (LACT_OPT_KEEP_PREACTIVATIONS 1 / 0): the recomputed products run over the same K-steps in the same order, so
    the output and every gradient have the same bits -- except the learning-rate gradients, fp32 sums over a token's
    hidden units that the two kernels take over tiles of different width (order of an fp32 sum: <= 1e-6)."""
    say("keep / recompute", b, L, d, dh, C, muon)
    from lact_amd import _lib
    inp = problem(b, L, d, dh, seed=56, act=torch.bfloat16)
    go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(9)).bfloat16().to(DEV)

    def run():
        t = clone_to(inp, DEV)
        out = T.block_causal_lact_swiglu(*args9(t), C, muon, t["momentum"])
        g = grads_of(out, t, go)
        torch.cuda.synchronize()
        return out, g
    L_ = _lib.lib()
    prev = L_.lact_set_option(_lib.OPT_KEEP_PREACTIVATIONS, 1)
    try:
        o1, g1 = run()
        L_.lact_set_option(_lib.OPT_KEEP_PREACTIVATIONS, 0)
        o0, g0 = run()
    finally:
        L_.lact_set_option(_lib.OPT_KEEP_PREACTIVATIONS, prev)
    assert torch.equal(o1, o0)
    for n in g0:
        if n in ("lr0", "lr1", "lr2"):
            assert O.rel_l2(g1[n], g0[n]) <= 1e-6, (n, O.rel_l2(g1[n], g0[n]))
        else:
            assert torch.equal(g1[n], g0[n]), (n, O.rel_l2(g1[n], g0[n]))


@pytest.mark.parametrize("chunks", [2, 3])
@pytest.mark.parametrize("b,d,dh", [(5, 384, 192), (2, 384, 384), (4, 384, 384), (3, 256, 128),
                                    (2, 768, 1536)])   # the video model's head: 32 blocks per matrix, a whole XCD per group
def test_fused_newton_schulz_is_bit_identical(b, d, dh, chunks):
    """All Newton-Schulz iterations of an update as one kernel with per-matrix barriers (rows, columns multiples
    of 192) against three GEMM launches per iteration: same tile code, same K order, and the dot product of the
    normalisation's backward summed over the same tiles in the same order on both paths -- so the same bits in the
    output AND in every gradient, with one update (chunks = 2) and with two chained ones (chunks = 3), with the apply
    steps running beside them on the second stream.  A stale tile or a missed barrier in the fused kernel shows here
    at any size.  Only d loss / d momentum (a handful of fp32 dot products <g, M_prev>, summed per tile by one path and
    per flat chunk by the other) may differ, by the order of an fp32 sum."""
    say("fused Newton-Schulz on/off", b, d, dh, "chunks", chunks)
    from lact_amd import _lib
    # (5, 384, 192): w1 is held transposed ([192, 384]), 15 matrices = a partial group of 8, 192-tiles;
    # (2, 384, 384), (4, 384, 384): few matrices -> 128 x 96 tiles, 12 blocks per matrix, one or two groups per XCD;
    # (3, 256, 128): only 128-tiles fit
    L, C = chunks * 256, 256
    inp = problem(b, L, d, dh, seed=91, act=torch.bfloat16)
    go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(6)).bfloat16().to(DEV)

    def run():
        res = []
        for _ in range(2):
            t = clone_to(inp, DEV)
            out = T.block_causal_lact_swiglu(*args9(t), C, True, t["momentum"])
            res.append((out, grads_of(out, t, go)))
        torch.cuda.synchronize()
        return res
    L_ = _lib.lib()
    prev = L_.lact_set_option(_lib.OPT_FUSED_NEWTON_SCHULZ, 1)
    try:
        on = run()
        L_.lact_set_option(_lib.OPT_FUSED_NEWTON_SCHULZ, 0)
        off = run()
    finally:
        L_.lact_set_option(_lib.OPT_FUSED_NEWTON_SCHULZ, prev)
    for (o1, g1), (o0, g0) in zip(on, off):
        assert torch.isfinite(o1.float()).all()
        assert torch.equal(o1, o0)
        for n in g0:
            assert torch.isfinite(g1[n].float()).all(), n
            if n == "momentum":
                if float(g0[n].float().norm()) > 0:
                    assert O.rel_l2(g1[n], g0[n]) < 1e-5, (n, O.rel_l2(g1[n], g0[n]))
                else:
                    assert float(g1[n].float().norm()) == 0.0
                continue
            assert torch.equal(g1[n], g0[n]), (n, O.rel_l2(g1[n], g0[n]))
    assert all(torch.equal(on[0][1][n], on[1][1][n]) for n in on[0][1])     # and each path repeats its own bits


# ---- fused-kernel variant (ttt_operation_fused_kernel.py): stacked Muon, eps inside the sqrt -------------
def fused_variant_pair(C, use_muon, prenorm):
    hf = T.prenorm_block_causal_lact_swiglu_fused_kernel_triton if prenorm else T.postnorm_block_causal_lact_swiglu_fused_kernel_triton
    of = O.prenorm_block_causal_lact_swiglu_fused_kernel_triton if prenorm else O.postnorm_block_causal_lact_swiglu_fused_kernel_triton
    return (lambda t: hf(*args9(t), C, use_muon, t["momentum"]),
            lambda t, num: of(*args9(t), C, use_muon, t["momentum"], num=num))


@pytest.mark.parametrize("b,L,d,dh,C,prenorm", [
    (2, 3 * 64 + 5, 64, 64, 64, False),       # stacked [128, 64]: held transposed
    (2, 2 * 96 + 17, 128, 64, 96, True),      # stacked [128, 128]: square; w1 [128, 64] transposed
    (2, 2 * 64 + 9, 256, 64, 64, False),      # stacked [128, 256]: as it lies
    (2, 3 * 128, 384, 384, 128, False)])      # 760M shape: stacked [768, 384] -> fused kernel on [384, 768]
def test_fused_variant_exact_arithmetic(b, L, d, dh, C, prenorm):
    """fp32 activations + fp32 Newton-Schulz against the float64 oracle: pins the stacked orthogonalisation
    (forward and backward, every layout case) and the eps-inside-sqrt renorm with its backward."""
    say("fused variant exact", b, L, d, dh, C, prenorm)
    inp = problem(b, L, d, dh, 19, torch.float32, momentum=True, lr_shift=-1.0)
    hip, orc = fused_variant_pair(C, True, prenorm)
    g = clone_to(inp, DEV)
    with ops.newton_schulz_mode(ops.NS_FP32):
        out = hip(g)
    go = torch.randn(out.shape, generator=torch.Generator().manual_seed(3))
    res = {"out": out, **grads_of(out, g, go.to(DEV))}
    c64 = clone_to(inp, "cpu", dtype_map=lambda t: torch.float64)
    o64 = orc(c64, EXACT)
    ref = {"out": o64, **grads_of(o64, c64, go.double())}
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < 1e-3


def test_fused_variant_small_rows_separate_the_eps_conventions():
    """Weights with tiny rows (|row|^2 ~ eps): the two renorm conventions differ by tens of percent there, so
    agreement with the oracle at 1e-3 shows the kernel has eps where the fused variant has it."""
    say("fused variant tiny rows")
    b, L, d, dh, C = 2, 2 * 64 + 3, 64, 64, 64
    inp = problem(b, L, d, dh, 23, torch.float32, momentum=False, lr_shift=-9.0)
    for n in ("w0", "w1", "w2"):
        inp[n] = inp[n] * 3e-3
    hip, orc = fused_variant_pair(C, False, False)
    res, ref = run_both(hip, orc, inp, PLAIN)
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < 1e-3
    other = O.block_causal_lact_swiglu(*args9(clone_to(inp, "cpu", grad=False)), C, False, None, num=PLAIN)
    assert O.rel_l2(ref["out"][:, C:], other[:, C:]) > 0.02


@pytest.mark.parametrize("b,L,d,dh,C,prenorm", [(2, 3 * 64 + 5, 64, 64, 64, False), (4, 1024, 384, 384, 512, False),
                                                (3, 3 * 256, 128, 256, 256, True)])
def test_fused_variant_bf16_muon(b, L, d, dh, C, prenorm):
    say("fused variant bf16 muon", b, L, d, dh, C, prenorm)
    inp = problem(b, L, d, dh, 29, torch.bfloat16, momentum=True)
    res, ref, r64, floors = run_both(*fused_variant_pair(C, True, prenorm), inp, AC, ref64=True, floor=True)
    assert_within_order_floor(res, ref, floors, "fused-variant", r64)
