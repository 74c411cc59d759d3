"""The entry point that allocates nothing (lact_newton_schulz_static: workspace in a fixed device array) against
lact_newton_schulz with a caller workspace, through the C ABI.  Same kernels in the same order, so the same bits."""
import ctypes
import sys

import pytest
import torch

from lact_amd import _lib
from oracle import lact_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _coeffs(co):
    flat = [float(x) for tr in co for x in tr]
    return (ctypes.c_float * max(1, len(flat)))(*flat)


def _both(L, G, co, mode):
    n, rows, cols = G.shape
    g = G.to(DEV).contiguous()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    arr = _coeffs(co)
    ws = torch.empty(L.lact_newton_schulz_workspace_bytes(n, rows, cols, len(co)), dtype=torch.uint8, device=DEV)
    want = torch.full_like(g, float("nan"))
    _lib.check(L.lact_newton_schulz(n, rows, cols, _ptr(g), _ptr(want), len(co), arr, mode, _ptr(ws), stream))
    got = torch.full_like(g, float("nan"))
    _lib.check(L.lact_newton_schulz_static(n, rows, cols, _ptr(g), _ptr(got), len(co), arr, mode, stream))
    torch.cuda.synchronize()
    return got, want


def test_static_workspace_newton_schulz_matches_the_workspace_entry_point():
    L = _lib.lib()
    assert L.lact_newton_schulz_static_capacity() == 32 << 20
    gen = torch.Generator().manual_seed(17)
    # two calls in a row on the same array, the second smaller (what the first left behind must not matter)
    for (n, rows, cols, kind, steps, mode) in [(3, 384, 384, "llm", 5, 0), (2, 64, 128, "classic", 3, 0), (2, 40, 24, "llm", 5, 1),
                                               (1, 128, 256, "classic", 5, 2)]:
        print("static newton_schulz", n, rows, cols, kind, steps, mode)
        sys.stdout.flush()
        G = torch.randn(n, rows, cols, generator=gen)
        co = O.ns_coeff_table(kind, steps)
        got, want = _both(L, G, co, mode)
        assert torch.isfinite(got).all() and torch.equal(got, want)          # bit for bit
        ref = O.newton_schulz(G.double(), co, O.Numerics(autocast=False, ns_dtype=None))
        assert O.rel_l2(got, ref) < 5e-2                                     # and it is Newton-Schulz
    # a shape beyond the array is refused with a message, and nothing runs
    n, rows, cols = 8, 1024, 1024
    assert L.lact_newton_schulz_workspace_bytes(n, rows, cols, 5) > L.lact_newton_schulz_static_capacity()
    g = torch.zeros(1, device=DEV)
    rc = L.lact_newton_schulz_static(n, rows, cols, _ptr(g), _ptr(g), 5, _coeffs(O.NS5_COEFFS), 0,
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc != 0 and b"static workspace holds" in L.lact_last_error()


def test_static_entry_point_allocates_nothing_and_replays_from_a_graph():
    """What the entry point exists for: after one warm-up call (which looks up the array's address and sets kernel
    attributes -- do that outside a capture), a call changes neither the device's free memory nor torch's allocator
    counters, and the call captured into a HIP graph replays to the same bits, several times, with eager work between
    the replays."""
    L = _lib.lib()
    gen = torch.Generator().manual_seed(29)
    n, rows, cols, co, mode = 3, 192, 384, O.ns_coeff_table("llm", 5), 0
    G = torch.randn(n, rows, cols, generator=gen)
    got, want = _both(L, G, co, mode)                       # warm-up of both entry points
    assert torch.equal(got, want)
    g = G.to(DEV).contiguous()
    out = torch.full_like(g, float("nan"))
    arr = _coeffs(co)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(L.lact_newton_schulz_static(n, rows, cols, _ptr(g), _ptr(out), len(co), arr, mode, stream))
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
    assert torch.equal(out, want)
    # captured: the call records kernels only (no allocation, no memset)
    out_g = torch.full_like(g, float("nan"))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check(L.lact_newton_schulz_static(n, rows, cols, _ptr(g), _ptr(out_g), len(co), arr, mode, s))
    torch.cuda.current_stream().wait_stream(side)
    for i in range(3):
        out_g.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, want), i
        # eager work of the program's own between the replays, on the same array
        got2, want2 = _both(L, torch.randn(2, 64, 128, generator=gen), O.ns_coeff_table("classic", 3), 0)
        assert torch.equal(got2, want2)
