"""Writes tests/golden/bidirectional_muon_cpu_fp32.npz.

The one statement of the hot path that no closed form pins against a mis-reading is the
bidirectional layer's Muon assignment (minimal_implementations/bidirectional_lact_layer.py:139-146:
the orthogonalised gradient overwrites the weight, then the raw gradient is added).  This script
loads that single reference file by path, in the build container only, with torch.compile
disabled, runs `bidirectional_lact_swiglu` on small seeded fp32 CPU inputs, and stores inputs and
outputs.  The fixture travels; the reference does not.

Usage (build container only):  TORCH_COMPILE_DISABLE=1 python tests/golden/make_bidirectional_golden.py
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
    for tag, (b, L, d, dh, seed, use_muon) in {
        "muon": (2, 96, 16, 24, 7, True),
        "nomuon": (2, 96, 16, 24, 8, False),
        "square": (1, 128, 32, 32, 9, True),
    }.items():
        g = torch.Generator().manual_seed(seed)
        rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
        q, k, v = rn(b, L, d), rn(b, L, d), rn(b, L, d)
        q = q / q.norm(dim=-1, keepdim=True)
        k = k / k.norm(dim=-1, keepdim=True)
        w0, w2, w1 = rn(b, dh, d) / d ** 0.5, rn(b, dh, d) / d ** 0.5, rn(b, d, dh) / dh ** 0.5
        lr0, lr1, lr2 = (torch.nn.functional.softplus(rn(b, L, 1)) * 1e-2 for _ in range(3))
        with torch.no_grad():
            o = mod.bidirectional_lact_swiglu(w0, w1, w2, q, k, v, lr0, lr1, lr2, use_muon)
        for name, t in dict(w0=w0, w1=w1, w2=w2, q=q, k=k, v=v, lr0=lr0, lr1=lr1, lr2=lr2, o=o).items():
            out[f"{tag}.{name}"] = t.numpy()
        out[f"{tag}.use_muon"] = np.array(use_muon)
    np.savez_compressed(os.path.join(HERE, "bidirectional_muon_cpu_fp32.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    sys.exit(main())
