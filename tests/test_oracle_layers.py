"""Pins the CPU restatement of the layer classes (oracle/lact_layers_oracle.py): golden vectors written from the
reference's own BidirectionalLaCTSwiGLU on the CPU (tests/golden/bidirectional_layer_cpu_fp32.npz), and
closed-form checks for what the causal layer adds (attention window, per-head gate, momentum head, q/k rescale)."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import lact_layers_oracle as LO
from oracle import lact_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden", "bidirectional_layer_cpu_fp32.npz")
PLAIN = O.Numerics(autocast=False)


def load_case(tag):
    z = np.load(GOLD)
    kw = {k.split(".kw.")[1]: z[k].item() for k in z.files if k.startswith(tag + ".kw.")}
    params = {k.split(".param.")[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(tag + ".param.")}
    grads = {k.split(".grad.")[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(tag + ".grad.")}
    t = lambda n: torch.from_numpy(z[f"{tag}.{n}"])
    return kw, params, grads, t("x"), t("go"), t("y"), t("dx")


@pytest.mark.parametrize("tag", ["muon", "plain"])
def test_bidirectional_layer_matches_reference_golden(tag):
    kw, params, grads, x, go, y, dx = load_case(tag)
    layer = LO.BidirectionalLaCTSwiGLU(num=PLAIN, **kw)
    missing = layer.load_state_dict(params, strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys       # same parameter names as the reference
    x = x.clone().requires_grad_(True)
    out = layer(x)
    out.backward(go)
    # the reference runs Newton-Schulz in bf16 on the CPU as well; same arithmetic here, so the match is tight
    tol = 2e-2 if kw["use_muon"] else 1e-5
    assert O.rel_l2(out, y) < tol
    assert O.rel_l2(x.grad, dx) < (5e-2 if kw["use_muon"] else 1e-4)
    for n, p in layer.named_parameters():
        assert O.rel_l2(p.grad, grads[n]) < (5e-2 if kw["use_muon"] else 1e-4), n


def test_sliding_window_attention_window_and_limits():
    g = torch.Generator().manual_seed(0)
    b, l, h, d = 2, 12, 3, 4
    q, k, v = (torch.randn(b, l, h, d, generator=g, dtype=torch.float64) for _ in range(3))
    # window 1: every query sees only itself -> output is v
    assert torch.allclose(LO.sliding_window_attention(q, k, v, 1), v, atol=1e-12)
    # window >= l equals plain causal attention (torch's own)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True).transpose(1, 2)
    assert torch.allclose(LO.sliding_window_attention(q, k, v, l), ref, atol=1e-10)
    assert torch.allclose(LO.sliding_window_attention(q, k, v, None), ref, atol=1e-10)
    # window W: changing a key/value more than W-1 positions back does not move the output row
    W = 4
    o1 = LO.sliding_window_attention(q, k, v, W)
    k2, v2 = k.clone(), v.clone()
    k2[:, 3] += 5.0
    v2[:, 3] -= 5.0
    o2 = LO.sliding_window_attention(q, k2, v2, W)
    assert torch.allclose(o1[:, 3 + W:], o2[:, 3 + W:], atol=1e-12) and not torch.allclose(o1[:, 3:3 + W], o2[:, 3:3 + W])


def test_causal_layer_composition():
    """With the fast-weight branch silenced (zero gate: ttt_scale_proj weight and bias zero -> silu(0) = 0) the layer
    is o_proj(attention); with the value third of to_qkv zeroed the attention branch vanishes and the layer is
    o_proj(gate * o_norm(op)): each branch is checked against an independent composition."""
    torch.manual_seed(3)
    dim, hd, ahd, L, B = 32, 16, 8, 40, 2
    layer = LO.CausalLaCTSwiGLUWithSlidingWindowAttn(dim, hd, ahd, lact_chunk_size=16, window_size=8, use_muon=False,
                                                     num=PLAIN).double()
    with torch.no_grad():
        layer.qk_scale.uniform_(0.5, 1.5)
        layer.qk_offset.uniform_(-0.2, 0.2)
    x = torch.randn(B, L, dim, dtype=torch.float64)
    with torch.no_grad():
        keep_w, keep_b = layer.ttt_scale_proj.weight.clone(), layer.ttt_scale_proj.bias.clone()
        layer.ttt_scale_proj.weight.zero_(); layer.ttt_scale_proj.bias.zero_()
        y = layer(x)
        qkv = layer.to_qkv(x)
        aq, ak, av = qkv.chunk(3, dim=-1)
        aq = aq * layer.qk_scale[:, 0] + layer.qk_offset[:, 0]
        ak = ak * layer.qk_scale[:, 1] + layer.qk_offset[:, 1]
        sh = lambda t: t.reshape(B, L, dim // ahd, ahd).transpose(1, 2)
        i = torch.arange(L)
        band = (i[None, :] <= i[:, None]) & (i[None, :] >= i[:, None] - 7)
        att = F.scaled_dot_product_attention(sh(aq), sh(ak), sh(av), attn_mask=band).transpose(1, 2).reshape(B, L, dim)
        assert torch.allclose(y, layer.o_proj(att), atol=1e-10)
        # fast-weight branch alone: with the value third of to_qkv zeroed the attention output is zero, and so
        # are the operation's v, hence every fast-weight gradient: the op reduces to f_w(q) with the initial weights
        layer.ttt_scale_proj.weight.copy_(keep_w); layer.ttt_scale_proj.bias.copy_(keep_b)
        layer.to_qkv.weight[2 * dim:].zero_()
        layer.o_norm.weight.uniform_(0.5, 1.5)
        y = layer(x)
        H = dim // hd
        qh = F.silu(layer.to_qkv(x))[..., :dim].reshape(B, L, H, hd)
        qh = qh / (qh.norm(dim=-1, keepdim=True) + 1e-5)
        rows = []
        for h in range(H):
            hid = F.silu(qh[:, :, h] @ layer.w0[h].T) * (qh[:, :, h] @ layer.w2[h].T)
            o = hid @ layer.w1[h].T
            o = o * torch.rsqrt((o * o).mean(dim=-1, keepdim=True) + 1e-5) * layer.o_norm.weight
            rows.append(o * F.silu(layer.ttt_scale_proj(x)[..., h:h + 1]))
        ref = layer.o_proj(torch.cat(rows, dim=-1))
        assert torch.allclose(y[:, :16], ref[:, :16], atol=1e-10)     # first chunk: the initial weights exactly
        assert O.rel_l2(y, ref) < 1e-3                                 # later chunks: only the renorm's eps moves the weights


def test_causal_layer_momentum_head_reaches_the_operation():
    """The momentum head (sigmoid of a linear map, one scalar per token and head) must enter the operation per
    head: forcing it to a constant through the bias reproduces the operation called with that constant."""
    torch.manual_seed(4)
    dim, hd, ahd, L, B = 32, 16, 8, 48, 2
    layer = LO.CausalLaCTSwiGLUWithSlidingWindowAttn(dim, hd, ahd, lact_chunk_size=16, window_size=8, use_muon=False,
                                                     use_o_norm=False, base_lr=1.0, num=PLAIN).double()
    x = torch.randn(B, L, dim, dtype=torch.float64)
    with torch.no_grad():
        layer.momentum_proj[0].weight.zero_()
        layer.momentum_proj[0].bias.copy_(torch.tensor([0.3, -1.2], dtype=torch.float64))   # per head
        y1 = layer(x)
        layer.momentum_proj[0].bias.zero_()
        y0 = layer(x)
        assert O.rel_l2(y1[:, 32:], y0[:, 32:]) > 1e-4         # momentum matters from the third chunk on
        assert torch.allclose(y1[:, :32], y0[:, :32], atol=1e-12)   # ... and not before (first update has no state)


EXACT = O.Numerics(autocast=False, ns_dtype=None)


def _nvs_layer(steps=0):
    torch.manual_seed(5)
    layer = LO.FastWeightGluMLPMultihead(dim=24, head_dim=8, inter_multi=2, bias=True, base_lr=0.02,
                                         muon_update_steps=steps, num=EXACT).double()
    with torch.no_grad():
        layer.o_norm.weight.uniform_(0.5, 1.5)
        layer.lr_fc.weight.mul_(3.0)       # rates that differ visibly between heads and between the three matrices
    return layer


def test_nvs_layer_against_per_head_composition():
    """lact_nvs/lact_ttt.py:200-241 written out head by head with explicit loops and index arithmetic: one update on
    rows [0, 12), then an apply on rows [4, 20) (Newton-Schulz with 0 iterations = Frobenius normalisation).  A wrong
    rate layout ('(h lrs)' for '(lrs h)'), a wrong head split of qkv, transposed fast weights or a norm over the
    wrong axis all fail it."""
    layer = _nvs_layer()
    B, L, D, H, hd = 2, 20, 24, 3, 8
    x = torch.randn(B, L, D, dtype=torch.float64)
    order = [O.TTTOperator(0, 12, True, False), O.TTTOperator(4, 20, False, True)]
    with torch.no_grad():
        y, st = layer(x, {"ttt_op_order": order})
        qkv = F.silu(layer.to_qkv(x))
        lr = F.softplus(layer.lr_fc(x) + layer.base_lr_inv)
        heads = []
        for b in range(B):
            row = []
            for h in range(H):
                q = qkv[b, :, 0 * D + h * hd:0 * D + (h + 1) * hd]
                k = qkv[b, :, 1 * D + h * hd:1 * D + (h + 1) * hd]
                v = qkv[b, :, 2 * D + h * hd:2 * D + (h + 1) * hd]
                q = q / (q.norm(dim=1, keepdim=True) + 1e-5)
                k = k / (k.norm(dim=1, keepdim=True) + 1e-5)
                l0, l1, l2 = (lr[b, :, s * H + h:s * H + h + 1] for s in range(3))
                w0, w1, w2 = layer.w0[h], layer.w1[h], layer.w2[h]          # [d, dh], [dh, d], [d, dh]
                n0, n1, n2 = (w.norm(dim=0, keepdim=True) for w in (w0, w1, w2))
                ki, vi = k[:12], v[:12]
                g, hb = ki @ w0, ki @ w2
                hid = F.silu(g) * hb
                dh_ = vi @ w1.T
                dhb = dh_ * F.silu(g)
                sg = torch.sigmoid(g)
                dg = dh_ * hb * sg * (1 + g * (1 - sg))
                fro = lambda m: m / (m.norm() + 1e-7)
                w1n = w1 + fro((hid * l1[:12]).T @ vi)
                w0n = w0 + fro((ki * l0[:12]).T @ dg)
                w2n = w2 + fro((ki * l2[:12]).T @ dhb)
                w0n = w0n / (w0n.norm(dim=0, keepdim=True) + 1e-5) * n0
                w1n = w1n / (w1n.norm(dim=0, keepdim=True) + 1e-5) * n1
                w2n = w2n / (w2n.norm(dim=0, keepdim=True) + 1e-5) * n2
                assert torch.allclose(st["w0"][b * H + h], w0n, atol=1e-12)
                assert torch.allclose(st["w1"][b * H + h], w1n, atol=1e-12)
                o = (F.silu(q[4:20] @ w0n) * (q[4:20] @ w2n)) @ w1n
                o = o * torch.rsqrt((o * o).mean(dim=1, keepdim=True) + 1e-5) * layer.o_norm.weight
                row.append(o)
            heads.append(torch.cat(row, dim=1))
        ref = layer.c_proj(torch.stack(heads))
    assert y.shape == (B, 16, D)
    assert torch.allclose(y, ref, atol=1e-11)


def test_nvs_layer_carries_weights_through_info():
    """Update in one call and apply in the next with the returned weights == both in one call
    (lact_nvs/model.py:272-384 runs reconstruction and rendering that way)."""
    layer = _nvs_layer(steps=2)
    x = torch.randn(2, 20, 24, dtype=torch.float64)
    with torch.no_grad():
        y_both, st_both = layer(x, {"ttt_op_order": [O.TTTOperator(0, 12, True, False), O.TTTOperator(0, 20, False, True)]})
        _y, st = layer(x, {"ttt_op_order": [O.TTTOperator(0, 12, True, True)]})
        y2, st2 = layer(x, {"ttt_op_order": [O.TTTOperator(0, 20, False, True)], **st})
    assert torch.allclose(y2, y_both, atol=1e-12)
    for n in ("w0", "w1", "w2"):
        assert torch.equal(st2[n], st[n]) and torch.allclose(st[n], st_both[n], atol=1e-12)
    assert not torch.allclose(st["w0"], layer.w0.repeat(2, 1, 1), atol=1e-3)
