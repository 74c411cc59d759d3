"""GPU parity of the layer classes in lact_amd/layers.py (pre-/post-processing kernels + the operation through the
C ABI) against the CPU oracle layers (oracle/lact_layers_oracle.py) and the golden vectors written from the
reference's own bidirectional layer."""
import os
import sys

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from lact_amd import layers as HL
from lact_amd import ops
from oracle import lact_layers_oracle as LO
from oracle import lact_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
GOLD = os.path.join(os.path.dirname(__file__), "golden", "bidirectional_layer_cpu_fp32.npz")
PLAIN = O.Numerics(autocast=False)
AC = O.Numerics(autocast=True)
EXACT = O.Numerics(autocast=False, ns_dtype=None)


def run_pair(ref_layer, layer, x, go, use_muon):
    """Muon: exact arithmetic on both sides (fp32 Newton-Schulz on the GPU, float64 oracle), so that the comparison
    pins the wiring instead of drowning in bf16 Newton-Schulz noise."""
    if use_muon:
        ref = grads_and_out(ref_layer.double(), x.double(), go.double())
        with ops.newton_schulz_mode(ops.NS_FP32):
            res = grads_and_out(layer, x.to(DEV), go.to(DEV))
    else:
        ref = grads_and_out(ref_layer, x, go)
        res = grads_and_out(layer, x.to(DEV), go.to(DEV))
    return res, ref


def say(*a):
    print(*a)
    sys.stdout.flush()


def grads_and_out(layer, x, go):
    x = x.clone().requires_grad_(True)
    y = layer(x)
    y.backward(go.to(y.dtype))
    res = {"y": y.detach().float().cpu(), "dx": x.grad.float().cpu()}
    for n, p in layer.named_parameters():
        res["d." + n] = p.grad.detach().float().cpu()
    layer.zero_grad(set_to_none=True)
    return res


def compare(res, ref):
    return {n: O.rel_l2(res[n], ref[n]) for n in ref if float(ref[n].double().norm()) > 0}


# ---- kernels alone -----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,B,L,H,hd,l2", [(torch.float32, 2, 37, 3, 16, True), (torch.float32, 1, 5, 2, 520, False),
                                                (torch.bfloat16, 2, 64, 4, 128, True)])
def test_pre_kernel_against_torch(dtype, B, L, H, hd, l2):
    say("layer pre", dtype, B, L, H, hd, l2)
    g = torch.Generator().manual_seed(1)
    qkv = torch.randn(B, L, 3 * H * hd, generator=g).to(dtype)
    gos = [torch.randn(B * H, L, hd, generator=g).to(dtype) for _ in range(3)]

    def torch_ref(t):
        y = F.silu(t)
        q, k, v = LO._heads(y, 3, H, hd)
        if l2:
            q = (q / (q.float().norm(dim=-1, keepdim=True) + 1e-5)).to(t.dtype)
            k = (k / (k.float().norm(dim=-1, keepdim=True) + 1e-5)).to(t.dtype)
        return q, k, v
    a = qkv.double().requires_grad_(True) if dtype == torch.float32 else qkv.clone().requires_grad_(True)
    ref = torch_ref(a)
    torch.autograd.backward(ref, [go.to(a.dtype) for go in gos])
    b_ = qkv.to(DEV).requires_grad_(True)
    out = HL._PreFn.apply(b_, H, hd, l2)
    torch.autograd.backward(out, [go.to(DEV) for go in gos])
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for o, r in zip(out, ref):
        assert O.rel_l2(o.float().cpu(), r.float()) < tol
    assert O.rel_l2(b_.grad.float().cpu(), a.grad.float()) < tol


def test_lr_kernel_against_torch():
    say("layer lr")
    g = torch.Generator().manual_seed(2)
    B, L, H = 2, 33, 3
    raw = (torch.randn(B, L, 3 * H, generator=g) * 3).requires_grad_(True)
    mraw = torch.randn(B, L, H, generator=g).requires_grad_(True)
    base = float(O.inv_softplus(1e-2))
    lr = F.softplus(raw.double() + base)
    ref = list(LO._heads(lr.reshape(B, L, H, 3).permute(0, 1, 3, 2).reshape(B, L, -1), 3, H, 1)) + \
        [LO._heads(torch.sigmoid(mraw.double()), 1, H, 1)[0]]
    gos = [torch.randn(B * H, L, 1, generator=g) for _ in range(4)]
    torch.autograd.backward(ref, [t.double() for t in gos])
    a, m = raw.detach().to(DEV).requires_grad_(True), mraw.detach().to(DEV).requires_grad_(True)
    out = HL._LrFn.apply(a, m, H, base)
    torch.autograd.backward(out, [t.to(DEV) for t in gos])
    for o, r in zip(out, ref):
        assert O.rel_l2(o.cpu(), r) < 1e-6
    assert O.rel_l2(a.grad.cpu(), raw.grad) < 1e-5 and O.rel_l2(m.grad.cpu(), mraw.grad) < 1e-5
    out3 = HL._LrFn.apply(a.detach(), None, H, base)
    assert len(out3) == 3 and torch.equal(out3[1], out[1])


@pytest.mark.parametrize("dtype,B,L,H,hd,norm,gate", [(torch.float32, 2, 37, 3, 16, True, True), (torch.float32, 1, 9, 2, 520, True, False),
                                                      (torch.float32, 2, 20, 2, 32, False, True), (torch.bfloat16, 2, 64, 4, 128, True, True)])
def test_post_kernel_against_torch(dtype, B, L, H, hd, norm, gate):
    say("layer post", dtype, B, L, H, hd, norm, gate)
    g = torch.Generator().manual_seed(3)
    o = torch.randn(B * H, L, hd, generator=g).to(dtype)
    w = torch.rand(hd, generator=g) + 0.5
    graw = torch.randn(B, L, H, generator=g).to(dtype)
    go = torch.randn(B, L, H * hd, generator=g).to(dtype)
    ct = torch.float64 if dtype == torch.float32 else torch.float32

    def torch_ref(o_, w_, g_):
        t = o_
        if norm:
            t = t * torch.rsqrt((t * t).mean(dim=-1, keepdim=True) + 1e-5) * w_
        if gate:
            t = t * LO._heads(F.silu(g_), 1, H, 1)[0]
        return LO._unheads(t, B, H)
    a, wa, ga = (t.detach().clone().to(ct).requires_grad_(True) for t in (o, w, graw))
    ref = torch_ref(a, wa, ga)
    ref.backward(go.to(ct))
    b_, wb, gb = (t.detach().clone().to(DEV).requires_grad_(True) for t in (o, w, graw))
    y = HL._PostFn.apply(b_, wb if norm else None, gb if gate else None, B, H, norm, 1e-5)
    y.backward(go.to(DEV))
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    assert O.rel_l2(y.float().cpu(), ref.float()) < tol
    assert O.rel_l2(b_.grad.float().cpu(), a.grad.float()) < tol
    if norm:
        assert O.rel_l2(wb.grad.cpu(), wa.grad.float()) < tol
    if gate:
        assert O.rel_l2(gb.grad.float().cpu(), ga.grad.float()) < tol


def test_sliding_window_attention_blocks_against_oracle():
    say("sliding window attention")
    g = torch.Generator().manual_seed(4)
    b, l, h, d = 2, 75, 3, 16
    q, k, v = (torch.randn(b, l, h, d, generator=g) for _ in range(3))
    for W in (1, 8, 32, 75, 200, None):
        ref = LO.sliding_window_attention(q.double(), k.double(), v.double(), W)
        out = HL.sliding_window_attention(q.to(DEV), k.to(DEV), v.to(DEV), W)
        assert O.rel_l2(out.cpu(), ref) < 1e-5, W


# ---- whole layers ------------------------------------------------------------------------------------
def load_gold(tag):
    z = np.load(GOLD)
    kw = {k.split(".kw.")[1]: z[k].item() for k in z.files if k.startswith(tag + ".kw.")}
    params = {k.split(".param.")[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(tag + ".param.")}
    ref = {"d." + k.split(".grad.")[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(tag + ".grad.")}
    ref["y"], ref["dx"] = torch.from_numpy(z[f"{tag}.y"]), torch.from_numpy(z[f"{tag}.dx"])
    return kw, params, ref, torch.from_numpy(z[f"{tag}.x"]), torch.from_numpy(z[f"{tag}.go"])


@pytest.mark.parametrize("tag", ["plain", "muon"])
def test_bidirectional_layer_against_reference_golden(tag):
    """The reference's own BidirectionalLaCTSwiGLU, run on the CPU in fp32 (tests/golden/): same parameters, same
    input, output and every gradient.  head_dim 16 / 24 here, so the operation runs on its generic fp32 kernels."""
    say("bidirectional layer golden", tag)
    kw, params, ref, x, go = load_gold(tag)
    layer = HL.BidirectionalLaCTSwiGLU(**kw).to(DEV)
    layer.load_state_dict(params, strict=True)
    res = grads_and_out(layer, x.to(DEV), go.to(DEV))
    errs = compare(res, ref)
    say("  ", errs)
    if not kw["use_muon"]:
        assert max(errs.values()) < 2e-4
        return
    # Muon: bf16 Newton-Schulz on both sides, here on 16 x 24 matrices whose forward comes out without a single
    # rounding flip: the output meets the fp32 bound outright.
    assert errs["y"] < 2e-4
    # The gradients pass through the backward of the bf16 iteration.  The HIP backward is a closed form that rounds
    # each of its three products per iteration once; autograd rounds every partial product and every gradient
    # accumulation of the same iteration (about as many roundings, at other points), so the two are independent
    # realisations of the same bf16 noise, each as far from float64 arithmetic as the other.  Yardstick: the larger of
    # the order-only floor (oracle against itself, accumulation order changed, O.order_variants) and the oracle's own
    # distance from the float64 oracle, per entry.
    def oracle_run(num, dt=torch.float32):
        ol = LO.BidirectionalLaCTSwiGLU(num=num, **kw).to(dt)
        ol.load_state_dict({k_: v_.to(dt) for k_, v_ in params.items()}, strict=True)
        return grads_and_out(ol, x.to(dt), go.to(dt))
    base = oracle_run(PLAIN)
    f64 = oracle_run(EXACT, torch.float64)
    yard = compare(base, f64)
    for v in O.order_variants(PLAIN):
        for n, e in compare(oracle_run(v), base).items():
            yard[n] = max(yard[n], e)
    say("   yardstick", yard, "oracle vs reference", compare(base, ref), "hip vs f64", compare(res, f64))
    for n, e in errs.items():
        assert e <= 1.5 * yard[n] + 1e-3, (n, e, yard[n])


@pytest.mark.parametrize("use_muon,use_o_norm,qk_l2", [(False, True, True), (False, False, False), (True, True, True)])
def test_bidirectional_layer_against_oracle(use_muon, use_o_norm, qk_l2):
    say("bidirectional layer vs oracle", use_muon, use_o_norm, qk_l2)
    torch.manual_seed(11)
    kw = dict(dim=256, head_dim=64, inter_multi=2, use_o_norm=use_o_norm, qk_l2_norm=qk_l2, use_muon=use_muon, base_lr=1e-2)
    ref_layer = LO.BidirectionalLaCTSwiGLU(num=EXACT if use_muon else PLAIN, **kw)
    layer = HL.BidirectionalLaCTSwiGLU(**kw).to(DEV)
    layer.load_state_dict(ref_layer.state_dict(), strict=True)
    x, go = torch.randn(2, 200, 256), torch.randn(2, 200, 256)
    res, ref = run_pair(ref_layer, layer, x, go, use_muon)
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < (1e-3 if use_muon else 2e-4)


@pytest.mark.parametrize("use_muon,use_momentum,window", [(False, True, 32), (False, False, 500), (True, True, 64)])
def test_causal_layer_against_oracle(use_muon, use_momentum, window):
    say("causal layer vs oracle", use_muon, use_momentum, window)
    torch.manual_seed(12)
    kw = dict(dim=256, head_dim=128, attn_head_dim=32, lact_chunk_size=64, window_size=window, inter_multi=1,
              use_o_norm=True, use_momentum=use_momentum, use_muon=use_muon, base_lr=1e-2)
    ref_layer = LO.CausalLaCTSwiGLUWithSlidingWindowAttn(num=EXACT if use_muon else PLAIN, **kw)
    with torch.no_grad():
        ref_layer.qk_scale.uniform_(0.5, 1.5)
        ref_layer.qk_offset.uniform_(-0.2, 0.2)
        ref_layer.o_norm.weight.uniform_(0.5, 1.5)
    layer = HL.CausalLaCTSwiGLUWithSlidingWindowAttn(**kw).to(DEV)
    layer.load_state_dict(ref_layer.state_dict(), strict=True)
    x, go = torch.randn(2, 3 * 64 + 20, 256), torch.randn(2, 3 * 64 + 20, 256)
    res, ref = run_pair(ref_layer, layer, x, go, use_muon)
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < (1e-3 if use_muon else 3e-4)


def test_causal_layer_bf16_autocast():
    """bf16 autocast as in training: projections and the operation in bf16, rates in fp32; against the oracle layer
    under the same autocast policy on the CPU."""
    say("causal layer bf16 autocast")
    torch.manual_seed(13)
    kw = dict(dim=512, head_dim=128, attn_head_dim=64, lact_chunk_size=128, window_size=128, use_muon=False)
    ref_layer = LO.CausalLaCTSwiGLUWithSlidingWindowAttn(num=AC, **kw)
    layer = HL.CausalLaCTSwiGLUWithSlidingWindowAttn(**kw).to(DEV)
    layer.load_state_dict(ref_layer.state_dict(), strict=True)
    x, go = torch.randn(2, 400, 512), torch.randn(2, 400, 512)
    with torch.autocast("cpu", dtype=torch.bfloat16):
        ref = grads_and_out(ref_layer, x, go)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        res = grads_and_out(layer, x.to(DEV), go.to(DEV))
    errs = compare(res, ref)
    say("  ", errs)
    assert res["y"].shape == ref["y"].shape
    assert max(errs.values()) < 3e-2


@pytest.mark.parametrize("steps", [0, 3])
def test_nvs_layer_against_oracle(steps):
    """FastWeightGluMLPMultihead (lact_nvs/lact_ttt.py:150-258): a reconstruction call (update + apply) whose
    returned fast weights feed a rendering call (apply only); output of both calls, the carried weights and every
    gradient against the float64 oracle layer (Newton-Schulz in fp32 on the GPU: exact arithmetic on both sides)."""
    say("nvs layer vs oracle, muon steps", steps)
    torch.manual_seed(14)
    kw = dict(dim=256, head_dim=64, inter_multi=2, bias=True, base_lr=0.01, muon_update_steps=steps)
    ref_layer = LO.FastWeightGluMLPMultihead(num=EXACT, **kw)
    with torch.no_grad():
        ref_layer.o_norm.weight.uniform_(0.5, 1.5)
    layer = HL.FastWeightGluMLPMultihead(**kw).to(DEV)
    layer.load_state_dict(ref_layer.state_dict(), strict=True)
    ref_layer = ref_layer.double()
    x1, x2 = torch.randn(2, 160, 256), torch.randn(2, 72, 256)
    go1, go2 = torch.randn(2, 100, 256), torch.randn(2, 72, 256)
    order1 = [O.TTTOperator(0, 96, True, True), O.TTTOperator(96, 160, True, False), O.TTTOperator(60, 64, False, True)]
    order2 = [O.TTTOperator(0, 72, False, True)]

    def run(lay, a, b, ga, gb):
        a = a.clone().requires_grad_(True)
        b = b.clone().requires_grad_(True)
        y1, st = lay(a, {"ttt_op_order": order1})
        y2, st2 = lay(b, {"ttt_op_order": order2, **st})
        (y1 * ga.to(y1.dtype)).sum().add((y2 * gb.to(y2.dtype)).sum()).backward()
        res = {"y1": y1, "y2": y2, "w0": st["w0"], "w1": st["w1"], "w2": st["w2"], "dx1": a.grad, "dx2": b.grad}
        res.update({"d." + n: p.grad for n, p in lay.named_parameters()})
        res = {n: t.detach().float().cpu() for n, t in res.items()}
        lay.zero_grad(set_to_none=True)
        return res

    ref = run(ref_layer, x1.double(), x2.double(), go1.double(), go2.double())
    with ops.newton_schulz_mode(ops.NS_FP32):
        res = run(layer, x1.to(DEV), x2.to(DEV), go1.to(DEV), go2.to(DEV))
    errs = compare(res, ref)
    say("  ", errs)
    assert res["y1"].shape == (2, 100, 256) and res["y2"].shape == (2, 72, 256)
    assert max(errs.values()) < 1e-3


def test_bidirectional_and_nvs_layers_bf16_autocast():
    """The two other layers under bf16 autocast (projections and operation in bf16, rates in fp32), against the
    oracle layers under the same policy on the CPU."""
    say("bidirectional + nvs layers bf16 autocast")
    torch.manual_seed(15)
    kw = dict(dim=256, head_dim=128, inter_multi=1, use_muon=False)
    ref_layer = LO.BidirectionalLaCTSwiGLU(num=AC, **kw)
    layer = HL.BidirectionalLaCTSwiGLU(**kw).to(DEV)
    layer.load_state_dict(ref_layer.state_dict(), strict=True)
    x, go = torch.randn(2, 300, 256), torch.randn(2, 300, 256)
    with torch.autocast("cpu", dtype=torch.bfloat16):
        ref = grads_and_out(ref_layer, x, go)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        res = grads_and_out(layer, x.to(DEV), go.to(DEV))
    errs = compare(res, ref)
    say("  ", errs)
    assert max(errs.values()) < 3e-2

    kw = dict(dim=256, head_dim=128, inter_multi=2, bias=True, muon_update_steps=0)
    ref_nvs = LO.FastWeightGluMLPMultihead(num=AC, **kw)
    nvs_layer = HL.FastWeightGluMLPMultihead(**kw).to(DEV)
    nvs_layer.load_state_dict(ref_nvs.state_dict(), strict=True)
    order = [O.TTTOperator(0, 200, True, False), O.TTTOperator(200, 300, False, True)]
    with torch.autocast("cpu", dtype=torch.bfloat16), torch.no_grad():
        y_ref, st_ref = ref_nvs(x, {"ttt_op_order": order})
    with torch.autocast("cuda", dtype=torch.bfloat16), torch.no_grad():
        y, st = nvs_layer(x.to(DEV), {"ttt_op_order": order})
    e = {"y": O.rel_l2(y.float().cpu(), y_ref.float()), **{n: O.rel_l2(st[n].float().cpu(), st_ref[n].float()) for n in st}}
    say("  ", e)
    assert y.shape == (2, 100, 256) and max(e.values()) < 3e-2


def test_layer_under_activation_checkpointing():
    """torch.utils.checkpoint runs the layer's forward a second time inside the backward (lact_nvs/train.py:106-123
    wraps its blocks that way): same output and gradients as the plain call."""
    say("layer under activation checkpointing")
    from torch.utils.checkpoint import checkpoint
    torch.manual_seed(16)
    layer = HL.CausalLaCTSwiGLUWithSlidingWindowAttn(dim=256, head_dim=128, attn_head_dim=64, lact_chunk_size=128,
                                                     window_size=64, use_muon=True).to(DEV)
    x = torch.randn(2, 3 * 128 + 17, 256, device=DEV)
    go = torch.randn_like(x)
    plain = grads_and_out(layer, x, go)
    xc = x.clone().requires_grad_(True)
    y = checkpoint(layer, xc, use_reentrant=False)
    y.backward(go)
    assert torch.equal(y.detach().float().cpu(), plain["y"])
    assert torch.equal(xc.grad.float().cpu(), plain["dx"])
    for n, p in layer.named_parameters():
        assert torch.equal(p.grad.detach().float().cpu(), plain["d." + n]), n
