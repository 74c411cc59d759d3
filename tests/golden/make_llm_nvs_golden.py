"""Writes tests/golden/llm_nvs_cpu_fp32.npz: the reference's own block-causal operations
(lact_llm/lact_model/ttt_operation.py: block_causal_lact_swiglu, prenorm_block_causal_lact_swiglu) and its NVS
program (lact_nvs/lact_ttt.py: fast_weight_swish_glu_weight_norm_mini_batch_apply), run on the CPU in fp32 with
torch.compile disabled, on tiny seeded inputs: output, final weights (NVS) and the gradient of every input.

Both files depend on torch (and einops) only and are loaded by path, in the build container only.  The fixture
travels; the reference does not.  On the CPU the reference's autocast decorator does nothing, so these are its
no-autocast numerics: fp32 everywhere, Newton-Schulz in bf16.

Usage (build container only):  TORCH_COMPILE_DISABLE=1 python tests/golden/make_llm_nvs_golden.py
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
NAMES = ("w0", "w1", "w2", "q", "k", "v", "lr0", "lr1", "lr2", "momentum")


def load(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def inputs(b, L, d, dh, seed, momentum, transposed=False):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    q, k, v = rn(b, L, d), rn(b, L, d), rn(b, L, d)
    q = q / q.norm(dim=-1, keepdim=True)
    k = k / k.norm(dim=-1, keepdim=True)
    w0, w2, w1 = rn(b, dh, d) / d ** 0.5, rn(b, dh, d) / d ** 0.5, rn(b, d, dh) / dh ** 0.5
    if transposed:      # NVS layout: w0, w2 [b, d, dh]; w1 [b, dh, d]
        w0, w1, w2 = (w.transpose(1, 2).contiguous() for w in (w0, w1, w2))
    lr0, lr1, lr2 = (torch.nn.functional.softplus(rn(b, L, 1) - 1.0) for _ in range(3))
    t = dict(w0=w0, w1=w1, w2=w2, q=q, k=k, v=v, lr0=lr0, lr1=lr1, lr2=lr2)
    if momentum:
        t["momentum"] = torch.sigmoid(rn(b, L, 1) + 1.5)
    return {n: x.requires_grad_(True) for n, x in t.items()}


def main():
    os.environ.setdefault("TORCH_COMPILE_DISABLE", "1")
    llm = load("/root/reference/lact_llm/lact_model/ttt_operation.py", "_ref_ttt_operation")
    nvs = load("/root/reference/lact_nvs/lact_ttt.py", "_ref_lact_ttt")
    out = {}

    def record(tag, t, results, go_seed, meta):
        # loss = sum of <result, fixed random tensor> over every returned tensor
        g = torch.Generator().manual_seed(go_seed)
        gos = [torch.randn(r.shape, generator=g) for r in results]
        loss = sum((r.float() * go).sum() for r, go in zip(results, gos))
        names = [n for n in NAMES if n in t]
        grads = torch.autograd.grad(loss, [t[n] for n in names])
        for n in names:
            out[f"{tag}.in.{n}"] = t[n].detach().numpy()
        for n, gr in zip(names, grads):
            out[f"{tag}.grad.{n}"] = gr.numpy()
        for i, (r, go) in enumerate(zip(results, gos)):
            out[f"{tag}.out.{i}"] = r.detach().float().numpy()
            out[f"{tag}.go.{i}"] = go.numpy()
        for k_, v_ in meta.items():
            out[f"{tag}.meta.{k_}"] = np.array(v_)

    # b=2, L=3C+5, C=16, d=8, dh=16: three whole chunks and a ragged tail
    for tag, fn, muon, mom, prenorm in [
            ("llm_plain", llm.block_causal_lact_swiglu, False, False, 0),
            ("llm_momentum", llm.block_causal_lact_swiglu, False, True, 0),
            ("llm_muon", llm.block_causal_lact_swiglu, True, True, 0),
            ("llm_prenorm", llm.prenorm_block_causal_lact_swiglu, False, True, 1),
            ("llm_prenorm_muon", llm.prenorm_block_causal_lact_swiglu, True, True, 1)]:
        t = inputs(2, 3 * 16 + 5, 8, 16, seed=100 + len(out), momentum=mom)
        o = fn(t["w0"], t["w1"], t["w2"], t["q"], t["k"], t["v"], t["lr0"], t["lr1"], t["lr2"], 16, muon, t.get("momentum"))
        record(tag, t, [o], 5, dict(chunk=16, use_muon=muon, prenorm=prenorm))
    # NVS programs: update on the first rows then apply on the rest; one operator that updates and applies; two updates
    for tag, order, steps in [
            ("nvs_update_then_apply", [(0, 40, True, False), (40, 56, False, True)], 0),
            ("nvs_update_and_apply_muon", [(0, 56, True, True)], 5),
            ("nvs_two_updates_muon", [(0, 24, True, False), (24, 48, True, True), (0, 56, False, True)], 3)]:
        t = inputs(2, 56, 8, 16, seed=200 + len(out), momentum=False, transposed=True)
        ops = [nvs.TTTOperator(*o) for o in order]
        res = nvs.fast_weight_swish_glu_weight_norm_mini_batch_apply(
            t["w0"], t["w1"], t["w2"], t["q"], t["k"], t["v"], t["lr0"], t["lr1"], t["lr2"], ops, muon_update_steps=steps)
        record(tag, t, list(res), 6, dict(order=np.array(order, dtype=np.int64), steps=steps))
    np.savez_compressed(os.path.join(HERE, "llm_nvs_cpu_fp32.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    sys.exit(main())
