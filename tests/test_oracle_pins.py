"""Pins the CPU oracle against things the mathematics or the reference's own output fixes.

Each test is chosen so that a plausible restatement mistake (dropped term, wrong lr on a weight,
transposed operand, wrong sign, wrong schedule bound) fails it.  No formula of the oracle is
retyped here: the checks are autograd identities, closed forms, invariants, brute force and the
golden vectors written from the reference on the CPU (tests/golden/).
"""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import lact_oracle as O

torch.manual_seed(0)
F64 = O.Numerics(autocast=False, ns_dtype=None)
PLAIN = O.Numerics(autocast=False)
GOLD = os.path.join(os.path.dirname(__file__), "golden", "bidirectional_muon_cpu_fp32.npz")


def rand_problem(b=2, L=40, d=8, dh=12, dtype=torch.float64, seed=0):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    w0, w2, w1 = rn(b, dh, d) / d ** 0.5, rn(b, dh, d) / d ** 0.5, rn(b, d, dh) / dh ** 0.5
    q, k, v = rn(b, L, d), rn(b, L, d), rn(b, L, d)
    lr0, lr1, lr2 = (F.softplus(rn(b, L, 1)) * 0.1 for _ in range(3))
    return w0, w1, w2, q, k, v, lr0, lr1, lr2


# ---- apply ------------------------------------------------------------------------------------
def test_apply_is_textbook_swiglu_mlp():
    w0, w1, w2, q, *_ = rand_problem()
    o = O.swiglu_apply(w0, w1, w2, q, F64)
    for i in range(q.shape[0]):
        ref = F.linear(F.silu(F.linear(q[i], w0[i])) * F.linear(q[i], w2[i]), w1[i])
        assert torch.allclose(o[i], ref, atol=1e-12)


# ---- fast-weight gradient: autograd identity with the lr that belongs to each weight ----------
def test_fast_weight_grads_are_autograd_of_lr_weighted_inner_product():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(seed=1)
    dw0, dw1, dw2 = O.fast_weight_grads(w0, w1, w2, k, v, lr0, lr1, lr2, F64)
    for w_idx, (lr, dw) in enumerate([(lr0, dw0), (lr1, dw1), (lr2, dw2)]):
        ws = [w.clone().requires_grad_(True) for w in (w0, w1, w2)]
        f = O.swiglu_apply(ws[0], ws[1], ws[2], k, F64)         # pinned above
        obj = (lr * (f * v).sum(-1, keepdim=True)).sum()
        (g,) = torch.autograd.grad(obj, ws[w_idx])
        assert torch.allclose(dw, g, atol=1e-10), w_idx
    # the three lrs are really distinct inputs: swapping two changes the result
    sw0, _, sw2 = O.fast_weight_grads(w0, w1, w2, k, v, lr2, lr1, lr0, F64)
    assert not torch.allclose(sw0, dw0) and not torch.allclose(sw2, dw2)


def test_silu_backprop_is_derivative_of_silu():
    x = torch.randn(50, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(50, dtype=torch.float64)
    (g,) = torch.autograd.grad(F.silu(x), x, dy)
    assert torch.allclose(O.silu_backprop(dy, x.detach()), g, atol=1e-12)


def test_l2_norm_and_inv_softplus():
    x = torch.randn(3, 5, 7)
    y = O.l2_norm(x)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1) / (x.norm(dim=-1) + 1e-5), atol=1e-6)
    assert y.dtype == x.dtype
    for val in (1e-3, 0.01, 1.0, 5.0):
        assert abs(F.softplus(torch.tensor(O.inv_softplus(val))).item() - val) < 1e-6
        assert abs(F.softplus(O.inv_softplus(torch.tensor(val))).item() - val) < 1e-6


# ---- Newton-Schulz ----------------------------------------------------------------------------
def _poly(s, coeffs):
    for a, b, c in coeffs:
        s = a * s + b * s ** 3 + c * s ** 5
    return s


def test_ns_coefficient_tables():
    assert len(O.NS5_COEFFS) == 5 and O.NS5_COEFFS[0] == (4.0848, -6.8946, 2.9270)
    assert O.NS5_COEFFS[4] == (2.8366, -3.0525, 1.2012)
    assert O.ns_coeff_table("classic", 3) == ((3.4445, -4.7750, 2.0315),) * 3
    assert O.ns_coeff_table("classic", 0) == ()


@pytest.mark.parametrize("shape", [(6, 6), (5, 9), (9, 5)])
def test_ns_acts_on_singular_values_by_the_quintic(shape):
    """X -> aX + (bA + cA^2)X with A = XX^T maps each singular value s to a s + b s^3 + c s^5 and
    keeps singular vectors; the Frobenius normalisation divides them by ||G||_F + 1e-7."""
    m, n = shape
    r = min(m, n)
    g = torch.Generator().manual_seed(3)
    U, _ = torch.linalg.qr(torch.randn(m, r, generator=g, dtype=torch.float64))
    V, _ = torch.linalg.qr(torch.randn(n, r, generator=g, dtype=torch.float64))
    s = torch.rand(r, generator=g, dtype=torch.float64) + 0.1
    G = (U * s) @ V.T
    out = O.newton_schulz(G[None], O.NS5_COEFFS, F64)[0]
    s0 = s / (s.norm() + 1e-7)
    ref = (U * _poly(s0, O.NS5_COEFFS)) @ V.T
    assert out.shape == G.shape
    assert torch.allclose(out, ref, atol=1e-10)
    # classic table, 3 steps
    out3 = O.newton_schulz(G[None], O.ns_coeff_table("classic", 3), F64)[0]
    assert torch.allclose(out3, (U * _poly(s0, [O.NS_CLASSIC] * 3)) @ V.T, atol=1e-10)
    # zero steps: normalisation only
    out0 = O.newton_schulz(G[None], (), F64)[0]
    assert torch.allclose(out0, G / (G.norm() + 1e-7), atol=1e-12)


def test_ns_invariances_and_bf16_default():
    G = torch.randn(3, 10, 6, dtype=torch.float64)
    a = O.newton_schulz(G, O.NS5_COEFFS, F64)
    assert torch.allclose(O.newton_schulz(3.7 * G, O.NS5_COEFFS, F64), a, atol=1e-9)
    assert torch.allclose(O.newton_schulz(G.transpose(1, 2), O.NS5_COEFFS, F64), a.transpose(1, 2), atol=1e-12)
    # singular values land in the advertised band
    sv = torch.linalg.svdvals(a)
    assert sv.max() < 1.6 and sv.min() > 0.3
    # default numerics: unconditional bf16 cast (ttt_operation.py:45) -> bf16 result on the CPU
    out = O.newton_schulz(G.float())
    assert out.dtype == torch.bfloat16
    assert O.rel_l2(out, a) < 0.1
    # autocast numerics: fp32 iterate (norm upcasts), bf16 matmuls
    out = O.newton_schulz(G.float(), O.NS5_COEFFS, O.Numerics(autocast=True))
    assert out.dtype == torch.float32 and O.rel_l2(out, a) < 0.05


# ---- renorm -----------------------------------------------------------------------------------
def test_renorm_row_norm_identity():
    w = torch.randn(2, 7, 5, dtype=torch.float64)
    n0 = torch.rand(2, 7, 1, dtype=torch.float64) + 0.5
    y = O.renorm(w, n0, F64)
    r = w.norm(dim=2, keepdim=True)
    assert torch.allclose(y.norm(dim=2, keepdim=True), n0 * r / (r + 1e-5), atol=1e-12)
    assert torch.allclose(y * (r + 1e-5) / n0, w, atol=1e-12)      # direction unchanged


# ---- schedule ---------------------------------------------------------------------------------
def _count(steps, kind):
    return sum(1 for s in steps if s.kind == kind)


@pytest.mark.parametrize("L,C", [(64, 16), (70, 16), (16, 16), (10, 16), (17, 16), (32768, 2048), (32760, 4680)])
def test_block_causal_schedule_counts(L, C):
    steps = O.block_causal_steps(L, C)
    n_chunks = max(1, math.ceil(L / C))
    assert _count(steps, O.APPLY) == n_chunks
    assert _count(steps, O.UPDATE) == n_chunks - 1
    covered = sorted((s.start, s.end) for s in steps if s.kind == O.APPLY)
    assert covered[0][0] == 0 and covered[-1][1] == L
    assert all(a[1] == b[0] for a, b in zip(covered, covered[1:]))
    # every update is preceded by the apply of the same chunk ("apply then update")
    for i, s in enumerate(steps):
        if s.kind == O.UPDATE:
            assert steps[i - 1] == O.Step(O.APPLY, s.start, s.end)


def test_short_sequence_is_plain_apply():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(L=12)
    o = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, chunk_size=16, use_muon=True,
                                   momentum=torch.full((2, 12, 1), 0.9, dtype=torch.float64), num=F64)
    assert torch.allclose(o, O.swiglu_apply(w0, w1, w2, q, F64), atol=1e-12)


def test_block_causality():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(L=56, seed=5)
    C = 16
    run = lambda k_, v_: O.block_causal_lact_swiglu(w0, w1, w2, q, k_, v_, lr0, lr1, lr2, C, True, None, num=F64)
    base = run(k, v)
    k2, v2 = k.clone(), v.clone()
    k2[:, 20] += 1.0
    v2[:, 20] -= 1.0                                   # token 20 lives in chunk 1 = [16, 32)
    pert = run(k2, v2)
    assert torch.allclose(base[:, :32], pert[:, :32], atol=1e-12)   # own chunk and earlier: unchanged
    assert (base[:, 32:48] - pert[:, 32:48]).abs().max() > 1e-6     # next chunk sees it
    # the last chunk's k, v are never used (apply-only)
    k3 = k.clone(); k3[:, 50] += 1.0
    assert torch.allclose(run(k3, v), base, atol=1e-12)


def test_momentum_matches_unrolled_recurrence():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(L=64, seed=6)
    C = 16
    mom = torch.rand(2, 64, 1, dtype=torch.float64)
    out = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, C, False, mom, num=F64)
    # brute force from the pinned stages
    ws = [w0, w1, w2]
    n0 = [w.norm(dim=2, keepdim=True) for w in ws]
    M = [torch.zeros_like(w) for w in ws]
    pieces = []
    for s in range(0, 64, C):
        pieces.append(O.swiglu_apply(ws[0], ws[1], ws[2], q[:, s:s + C], F64))
        if s + C >= 64:
            break
        dws = O.fast_weight_grads(ws[0], ws[1], ws[2], k[:, s:s + C], v[:, s:s + C],
                                  lr0[:, s:s + C], lr1[:, s:s + C], lr2[:, s:s + C], F64)
        mu = mom[:, s:s + C].sum(1, keepdim=True) / C
        M = [dw + mu * m for dw, m in zip(dws, M)]
        ws = [O.renorm(w + m, n, F64) for w, m, n in zip(ws, M, n0)]
    assert torch.allclose(out, torch.cat(pieces, 1), atol=1e-12)
    # momentum == 0 carries nothing; momentum None skips
    z = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, C, False, torch.zeros_like(mom), num=F64)
    n = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, C, False, None, num=F64)
    assert torch.allclose(z, n, atol=1e-12) and not torch.allclose(out, n, atol=1e-6)


def test_prenorm_differs_only_through_the_accumulator():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(L=64, seed=7)
    post = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, False, None, num=F64)
    pre = O.prenorm_block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, False, None, num=F64)
    # first two chunks see identical weights (one update from the same start); later ones differ
    assert torch.allclose(post[:, :32], pre[:, :32], atol=1e-12)
    assert (post[:, 32:] - pre[:, 32:]).abs().max() > 1e-8


def test_minimal_argument_order():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(L=48, seed=8)
    mom = torch.full((2, 48, 1), 0.5, dtype=torch.float64)
    a = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, True, mom, num=F64)
    b = O.block_causal_lact_swiglu_minimal(w0, w1, w2, q, k, v, lr0, lr1, lr2, mom, True, 16, num=F64)
    assert torch.equal(a, b)


# ---- NVS program: transposed layout, concatenated output --------------------------------------
def test_nvs_program_equals_llm_layout_on_transposed_weights():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(L=48, seed=9)
    prog = [O.TTTOperator(0, 32, True, False), O.TTTOperator(0, 48, False, True)]
    out, a0, a1, a2 = O.fast_weight_swish_glu_weight_norm_mini_batch_apply(
        w0.transpose(1, 2).contiguous(), w1.transpose(1, 2).contiguous(), w2.transpose(1, 2).contiguous(),
        q, k, v, lr0, lr1, lr2, prog, muon_update_steps=5, num=F64)
    ref, (b0, b1, b2), _ = O.run_program(w0, w1, w2, q, k, v, lr0, lr1, lr2,
                                         [O.Step(O.UPDATE, 0, 32), O.Step(O.APPLY, 0, 48)], num=F64,
                                         ns_coeffs=[O.NS_CLASSIC] * 5)
    assert out.shape == (2, 48, 8) and a0.shape == (2, 8, 12) and a1.shape == (2, 12, 8)
    assert torch.allclose(out, ref, atol=1e-12) and torch.allclose(a1.transpose(1, 2), b1, atol=1e-12)
    # update+apply in one operator applies the UPDATED weights; two applies are concatenated
    prog2 = [O.TTTOperator(0, 16, True, True), O.TTTOperator(16, 48, False, True)]
    out2, *_ = O.fast_weight_swish_glu_weight_norm_mini_batch_apply(
        w0.transpose(1, 2), w1.transpose(1, 2), w2.transpose(1, 2), q, k, v, lr0, lr1, lr2, prog2, 0, num=F64)
    assert out2.shape == (2, 48, 8)
    assert not torch.allclose(out2[:, :16], O.swiglu_apply(w0, w1, w2, q[:, :16], F64), atol=1e-6)


def test_ar_video_schedule_and_w_scale():
    steps = O.ar_video_steps(seq_len=60, mini_batch_size=10, update_length=60, update_every=20)
    assert steps[0] == O.Step(O.APPLY, 0, 10)
    assert steps[1:3] == [O.Step(O.UPDATE, 10, 20), O.Step(O.APPLY, 10, 30)]
    assert steps[-1] == O.Step(O.APPLY, 50, 60) and len(steps) == 7
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(L=60, seed=10)
    a = O.ar_fast_weight_swish_glu_weight_norm_mini_batch(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.5,
                                                         mini_batch_size=10, update_every=20, num=F64)
    b = O.ar_fast_weight_swish_glu_weight_norm_mini_batch(w0, w1, w2, q, k, v, 0.5 * lr0, 0.5 * lr1, 0.5 * lr2,
                                                         1.0, mini_batch_size=10, update_every=20, num=F64)
    assert len(a) == 4 and all(torch.allclose(x, y, atol=1e-12) for x, y in zip(a, b))
    # first block is untouched by any update
    assert torch.allclose(a[0][:, :10], O.swiglu_apply(w0, w1, w2, q[:, :10], F64), atol=1e-12)


# ---- golden vectors written from the reference (CPU, fp32, torch.compile disabled) ------------
@pytest.mark.parametrize("tag", ["muon", "nomuon", "square"])
def test_bidirectional_golden(tag):
    z = np.load(GOLD)
    t = {n: torch.from_numpy(z[f"{tag}.{n}"]) for n in ("w0", "w1", "w2", "q", "k", "v", "lr0", "lr1", "lr2", "o")}
    use_muon = bool(z[f"{tag}.use_muon"])
    o = O.bidirectional_lact_swiglu(t["w0"], t["w1"], t["w2"], t["q"], t["k"], t["v"], t["lr0"], t["lr1"],
                                    t["lr2"], use_muon, num=O.Numerics(autocast=False))
    assert o.dtype == t["o"].dtype
    # same ops, same dtypes, same order -> identical up to matmul blocking
    assert O.rel_l2(o, t["o"]) < 1e-5, O.rel_l2(o, t["o"])
    if use_muon:   # and the other reading of :139-146 does NOT reproduce the reference's output
        other = O.bidirectional_lact_swiglu(t["w0"], t["w1"], t["w2"], t["q"], t["k"], t["v"], t["lr0"],
                                            t["lr1"], t["lr2"], True, muon_mode="intended")
        assert O.rel_l2(other, t["o"]) > 1e-2


# ---- autocast numerics stay close to exact arithmetic; gradcheck of the whole op --------------
def test_autocast_numerics_track_fp64():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(b=2, L=96, d=32, dh=32, seed=11)
    q = q / q.norm(dim=-1, keepdim=True); k = k / k.norm(dim=-1, keepdim=True)
    mom = torch.full((2, 96, 1), 0.9, dtype=torch.float64)
    ref = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, 32, True, mom, num=F64)
    f = lambda t: t.float()
    out = O.block_causal_lact_swiglu(f(w0), f(w1), f(w2), q.bfloat16(), k.bfloat16(), v.bfloat16(),
                                     f(lr0), f(lr1), f(lr2), 32, True, f(mom), num=O.Numerics(autocast=True))
    assert out.dtype == torch.bfloat16
    assert O.rel_l2(out, ref) < 5e-2


def test_whole_op_gradcheck_fp64():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(b=1, L=20, d=4, dh=6, seed=12)
    mom = torch.rand(1, 20, 1, dtype=torch.float64)
    args = [t.clone().requires_grad_(True) for t in (w0, w1, w2, q, k, v, lr0, lr1, lr2, mom)]
    fn = lambda *a: O.block_causal_lact_swiglu(*a[:9], 8, True, a[9], num=F64)
    assert torch.autograd.gradcheck(fn, args, eps=1e-6, atol=1e-5, rtol=1e-4)


# ---- fused-kernel variant (ttt_operation_fused_kernel.py) -----------------------------------------
def test_fused_variant_orthogonalises_the_stacked_gradient():
    """One update, no renorm, exact arithmetic: cat(w0', w2') - cat(w0, w2) must be the quintic acting on the
    singular values of the STACKED gradient cat(dw0, dw2) / ||.||_F (one SVD of the [2dh, d] matrix), and
    w1' - w1 the same for dw1 alone.  Orthogonalising dw0 and dw2 separately fails this."""
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(b=2, L=24, d=6, dh=5)
    L = k.shape[1]
    steps = [O.Step(O.UPDATE, 0, L), O.Step(O.APPLY, 0, L)]
    _, (n0, n1, n2), _ = O.run_program(w0, w1, w2, q, k, v, lr0, lr1, lr2, steps, num=F64, ns_coeffs=O.NS5_COEFFS,
                                      weight_norm=False, stack_muon=True)
    dw0, dw1, dw2 = O.fast_weight_grads(w0, w1, w2, k, v, lr0, lr1, lr2, F64)

    def orth(G):
        U, s, Vh = torch.linalg.svd(G, full_matrices=False)
        return (U * _poly(s / (s.norm() + 1e-7), O.NS5_COEFFS)) @ Vh
    for i in range(w0.shape[0]):
        got = torch.cat([n0[i] - w0[i], n2[i] - w2[i]], dim=0)
        assert torch.allclose(got, orth(torch.cat([dw0[i], dw2[i]], dim=0)), atol=1e-9)
        assert torch.allclose(n1[i] - w1[i], orth(dw1[i]), atol=1e-9)
        separate = torch.cat([orth(dw0[i]), orth(dw2[i])], dim=0)
        assert not torch.allclose(got, separate, atol=1e-3)


def test_fused_variant_renorm_has_eps_inside_the_sqrt():
    """Row norms after y = x / sqrt(|x|^2 + eps) * n: |y| = n |x| / sqrt(|x|^2 + 1e-5); with |x|^2 ~ eps the two
    conventions differ by tens of percent, so the check separates them."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 4, 9, generator=g, dtype=torch.float64) * 1e-3
    n = torch.rand(2, 4, 1, generator=g, dtype=torch.float64) + 0.5
    y = O.renorm(x, n, F64, eps_in_sqrt=True)
    xn = x.norm(dim=2, keepdim=True)
    assert torch.allclose(y.norm(dim=2, keepdim=True), n * xn / torch.sqrt(xn ** 2 + 1e-5), rtol=1e-6)   # fp32 statistics
    assert torch.allclose(y / y.norm(dim=2, keepdim=True), x / xn, atol=1e-6)                            # direction kept
    y_out = O.renorm(x, n, F64)
    assert torch.allclose(y_out.norm(dim=2, keepdim=True), n * xn / (xn + 1e-5), rtol=1e-10)
    assert (y.norm(dim=2) / y_out.norm(dim=2) - 1).abs().min() > 0.05


def test_fused_variant_entry_points_share_schedule_and_differ_only_in_the_two_switches():
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(b=2, L=50, d=6, dh=5)
    mom = torch.sigmoid(torch.randn(2, 50, 1, dtype=torch.float64))
    # without Muon the post-norm variants differ only through eps placement: at these row norms (~1) by ~1e-5
    a = O.postnorm_block_causal_lact_swiglu_fused_kernel_triton(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, False, mom, num=F64)
    b_ = O.block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, False, mom, num=F64)
    assert a.shape == b_.shape and 0 < O.rel_l2(a, b_) < 1e-4
    # pre-norm without Muon: identical (eps stays outside, :322-327)
    a = O.prenorm_block_causal_lact_swiglu_fused_kernel_triton(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, False, mom, num=F64)
    b_ = O.prenorm_block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, False, mom, num=F64)
    assert torch.equal(a, b_)
    # with Muon the stacking changes the result visibly, the first chunk (no update yet) not at all
    a = O.prenorm_block_causal_lact_swiglu_fused_kernel_triton(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, True, mom, num=F64)
    b_ = O.prenorm_block_causal_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, 16, True, mom, num=F64)
    assert torch.equal(a[:, :16], b_[:, :16]) and O.rel_l2(a[:, 16:], b_[:, 16:]) > 1e-3


# ---- inference step with momentum states carried between calls ------------------------------------------
def test_carried_momentum_state_composes_and_is_the_heavy_ball_step():
    """ar_lact_swa_repeat_sp.py:197-339.  (1) Without weight norm the states and weights after two calls, each
    doing one update and handing its results to the next, equal one call doing both updates (a dropped or
    re-zeroed state fails).  (2) A call with a given state M adds exactly mean(momentum) * M to the step a call
    without state makes, on every weight, and returns step + that as the new state (wrong sign, wrong mean, a
    state applied to the wrong weight fail).  (3) States pass through untouched when nothing updates."""
    w0, w1, w2, q, k, v, lr0, lr1, lr2 = rand_problem(seed=5)
    mom = torch.sigmoid(torch.randn(2, 40, 1, dtype=torch.float64))
    fn = O.ar_fast_weight_swish_glu_weight_norm_mini_batch_inference_with_momentum
    kw = dict(num=F64)
    both = fn(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.7, 2, 24, True, False, 3, False, mom, None, None, None, True, **kw)
    one = fn(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.7, 1, 24, True, False, 3, False, mom, None, None, None, True, **kw)
    two = fn(one[1], one[2], one[3], q, k, v, lr0, lr1, lr2, 0.7, 1, 24, True, False, 3, False, mom, one[4], one[5],
             one[6], True, **kw)
    for a, b_ in zip(both, two):
        assert torch.allclose(a, b_, atol=1e-12)
    # (2): same weights, with and without a state
    M = [torch.randn_like(w) for w in (w0, w1, w2)]
    bare = fn(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.7, 1, 24, True, False, 3, False, mom, None, None, None, True, **kw)
    with_m = fn(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.7, 1, 24, True, False, 3, False, mom, M[0], M[1], M[2], True, **kw)
    mbar = mom[:, :24].mean(dim=1, keepdim=True)
    for j, w in enumerate((w0, w1, w2)):
        step = bare[1 + j] - w
        assert torch.allclose(bare[4 + j], step, atol=1e-12)                     # first state = first step
        assert torch.allclose(with_m[1 + j] - w, step + mbar * M[j], atol=1e-12)
        assert torch.allclose(with_m[4 + j], step + mbar * M[j], atol=1e-12)
    # (3)
    idle = fn(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.7, 1, 24, False, False, 3, True, mom, M[0], M[1], M[2], True, **kw)
    assert all(idle[4 + j] is M[j] for j in range(3)) and all(idle[1 + j] is w for j, w in enumerate((w0, w1, w2)))
    assert torch.allclose(idle[0], O.swiglu_apply(w0, w1, w2, q, F64), atol=1e-12)
    zeros = fn(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.7, 1, 24, False, False, 3, True, mom, None, None, None, True, **kw)
    assert all(float(zeros[4 + j].abs().max()) == 0.0 for j in range(3))
    off = fn(w0, w1, w2, q, k, v, lr0, lr1, lr2, 0.7, 1, 24, True, False, 3, True, None, None, None, None, False, **kw)
    assert off[4] is None and off[5] is None and off[6] is None


# ---- the order-only floor of the bf16 Muon path -------------------------------------------------------------
@pytest.mark.parametrize("b,L,d,dh,C", [(2, 3 * 64 + 5, 64, 64, 64), (2, 1024, 384, 384, 512)])
def test_order_only_floor_of_bf16_newton_schulz(b, L, d, dh, C):
    """How far the oracle moves when NOTHING changes but the order in which its bf16 GEMMs and its norms add their
    terms (same operands, same rounding points): float64 accumulation, K blocks of 16 ascending, K blocks of 64
    descending.  Without Muon that is the fp32 summation noise (below 1e-3 on every output); with Muon the
    Newton-Schulz iteration magnifies single bf16 rounding flips to about 1e-2 on the output -- the size of the
    north-star bf16 tolerance itself.  The GPU parity tests state their Muon bound as 1.5 x this floor, measured on
    their own inputs; here its size is pinned so that it cannot be inflated unnoticed (an order variant that also
    moved a rounding point would show up in the Muon-off leg, which must stay at summation-noise level)."""
    inp = O.make_inputs(b, L, d, dh, seed=7, act_dtype=torch.bfloat16, momentum_value=None)
    inp["momentum"] = torch.sigmoid(torch.randn(b, L, 1, generator=torch.Generator().manual_seed(106)) + 1.5)
    order = ("w0", "w1", "w2", "q", "k", "v", "lr0", "lr1", "lr2")
    steps = O.block_causal_steps(L, C)
    base = O.Numerics(autocast=True)
    for muon in (False, True):
        run = lambda num: O.run_program(*[inp[n] for n in order], steps, num=num, momentum=inp["momentum"],
                                        ns_coeffs=O.NS5_COEFFS if muon else None)
        ref_out, ref_w, _ = run(base)
        f_out, f_w = 0.0, 0.0
        for v in O.order_variants(base):
            out, ws, _ = run(v)
            f_out = max(f_out, O.rel_l2(out, ref_out))
            f_w = max(f_w, max(O.rel_l2(a, r) for a, r in zip(ws, ref_w)))
        print(f"order-only floor d={d} muon={muon}: output {f_out:.2e}, fast weights {f_w:.2e}")
        if muon:
            assert 3e-3 < f_out < 4e-2 and 3e-3 < f_w < 4e-2
        else:
            assert f_out < 1e-3 and f_w < 1e-4


# ---- golden vectors of the LLM operations and the NVS program, written from the reference (CPU, fp32) ---------
LLM_NVS_GOLD = os.path.join(os.path.dirname(__file__), "golden", "llm_nvs_cpu_fp32.npz")
LLM_TAGS = ("llm_plain", "llm_momentum", "llm_muon", "llm_prenorm", "llm_prenorm_muon")
NVS_TAGS = ("nvs_update_then_apply", "nvs_update_and_apply_muon", "nvs_two_updates_muon")


def load_llm_nvs_gold(tag):
    z = np.load(LLM_NVS_GOLD)
    pick = lambda kind: {k.split(f".{kind}.")[1]: z[k] for k in z.files if k.startswith(f"{tag}.{kind}.")}
    t = {n: torch.from_numpy(a) for n, a in pick("in").items()}
    grads = {n: torch.from_numpy(a) for n, a in pick("grad").items()}
    outs = [torch.from_numpy(a) for _, a in sorted(pick("out").items())]
    gos = [torch.from_numpy(a) for _, a in sorted(pick("go").items())]
    return t, outs, gos, grads, pick("meta")


def run_oracle_on_gold(tag, t, meta, num=PLAIN):
    t = {n: v.clone().requires_grad_(True) for n, v in t.items()}
    a = [t[n] for n in ("w0", "w1", "w2", "q", "k", "v", "lr0", "lr1", "lr2")]
    if tag.startswith("llm"):
        res = [O.block_causal_lact_swiglu(*a, int(meta["chunk"]), bool(meta["use_muon"]), t.get("momentum"), num=num,
                                          prenorm=bool(meta["prenorm"]))]
    else:
        order = [O.TTTOperator(int(s), int(e), bool(u), bool(ap)) for s, e, u, ap in meta["order"]]
        res = list(O.fast_weight_swish_glu_weight_norm_mini_batch_apply(*a, order, int(meta["steps"]), num=num))
    return t, res


@pytest.mark.parametrize("tag", LLM_TAGS + NVS_TAGS)
def test_llm_and_nvs_golden(tag):
    """tests/golden/make_llm_nvs_golden.py: ttt_operation.py:71-364 and lact_ttt.py:71-147 themselves, run on the CPU:
    output, returned weights and the gradient of every input.  Same library, same operations in the same order:
    the oracle has to reproduce them to fp32 round-off, Newton-Schulz in bf16 included."""
    t, outs, gos, grads, meta = load_llm_nvs_gold(tag)
    tt, res = run_oracle_on_gold(tag, t, meta)
    assert len(res) == len(outs)
    for r, o in zip(res, outs):
        assert r.shape == o.shape and O.rel_l2(r, o) < 1e-5, (tag, O.rel_l2(r, o))
    loss = sum((r.float() * go).sum() for r, go in zip(res, gos))
    names = list(grads)
    got = torch.autograd.grad(loss, [tt[n] for n in names])
    for n, g in zip(names, got):
        assert O.rel_l2(g, grads[n]) < 1e-5, (tag, n, O.rel_l2(g, grads[n]))
