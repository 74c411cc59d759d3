"""Compiles lact_amd/csrc into lact_amd/lib/liblact_hip.so for gfx950 with hipcc (cross-compiles
without a GPU).  Usage: python -m lact_amd.build"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "lact_api.hip")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "liblact_hip.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # A multiply and an add fuse only where one source expression writes them together.  HIP's default ("fast") also
    # fuses across statements and inlined calls, i.e. through __fmul_rn / __fadd_rn, which are plain operators in the
    # HIP headers: whether a product that the reference rounds as a tensor of its own (a * X before + B @ X,
    # ttt_operation.py:62; M * m before dw +, :174-176) got its own rounding then depended on how the surrounding
    # kernel was inlined -- the fused and the unfused Newton-Schulz backward differed in exactly that.
    "-ffp-contract=on",
    # the copy engine sets m0 in its own asm statements and names it as clobbered; no compiler-generated code in these
    # kernels uses m0 (no LDS-DMA builtins, no register-indexed moves, no messages)
    "-Wno-inline-asm",
]


def build(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + [SRC, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
