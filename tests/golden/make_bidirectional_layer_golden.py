"""Writes tests/golden/bidirectional_layer_cpu_fp32.npz.

Pins the layer class around the operation (projections, SiLU, per-head L2 norm, softplus learning rates with
the inverse-softplus offset, head layout, RMSNorm, output projection): loads the single reference file
minimal_implementations/bidirectional_lact_layer.py by path, in the build container only, with torch.compile
disabled, builds `BidirectionalLaCTSwiGLU` on the CPU in fp32 from a fixed seed, and stores its parameters, an
input, the output and the gradients of a fixed upstream gradient.  The fixture travels; the reference does not.

Usage (build container only):  TORCH_COMPILE_DISABLE=1 python tests/golden/make_bidirectional_layer_golden.py
"""
import importlib.util
import os
import sys

import numpy as np
import torch

REF = "/root/reference/minimal_implementations/bidirectional_lact_layer.py"
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    os.environ.setdefault("TORCH_COMPILE_DISABLE", "1")
    spec = importlib.util.spec_from_file_location("_ref_bidirectional", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)

    out = {}
    cases = {
        "muon": dict(dim=64, head_dim=16, inter_multi=1.5, use_o_norm=True, qk_l2_norm=True, use_muon=True, base_lr=1e-2),
        "plain": dict(dim=48, head_dim=24, inter_multi=1.0, use_o_norm=False, qk_l2_norm=False, use_muon=False, base_lr=3e-2),
    }
    for i, (tag, kw) in enumerate(cases.items()):
        torch.manual_seed(100 + i)
        layer = mod.BidirectionalLaCTSwiGLU(**kw).float()
        if kw["use_o_norm"]:
            with torch.no_grad():
                layer.o_norm.weight.uniform_(0.5, 1.5)
        B, L = 2, 80
        x = torch.randn(B, L, kw["dim"], requires_grad=True)
        go = torch.randn(B, L, kw["dim"])
        y = layer(x)
        y.backward(go)
        out[f"{tag}.x"], out[f"{tag}.go"], out[f"{tag}.y"], out[f"{tag}.dx"] = x.detach().numpy(), go.numpy(), y.detach().numpy(), x.grad.numpy()
        for n, p in layer.named_parameters():
            out[f"{tag}.param.{n}"] = p.detach().numpy()
            out[f"{tag}.grad.{n}"] = p.grad.numpy()
        for k_, v_ in kw.items():
            out[f"{tag}.kw.{k_}"] = np.array(v_)
    np.savez_compressed(os.path.join(HERE, "bidirectional_layer_cpu_fp32.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    sys.exit(main())
