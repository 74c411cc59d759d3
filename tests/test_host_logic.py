"""Host-side logic of the HIP library that needs no GPU: the XCD-aware block -> tile maps are bijections
(compiled and run as a host program), and the option switch validates its arguments."""
import os
import subprocess


from lact_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_tile_maps_cover_every_tile_once(tmp_path):
    src = os.path.join(ROOT, "tests", "host", "tilemap_check.hip")
    exe = str(tmp_path / "tilemap_check")
    cmd = ["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O1", "-std=c++17", "-Wno-inline-asm", src, "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "0 bad" in out.stdout


def test_set_option_round_trip_and_unknown_option():
    L = _lib.lib()
    for opt in (_lib.OPT_STREAM_OVERLAP, _lib.OPT_FUSED_NEWTON_SCHULZ):
        prev = L.lact_set_option(opt, 0)
        assert prev in (0, 1)
        assert L.lact_set_option(opt, 1) == 0
        assert L.lact_set_option(opt, prev) == 1
    assert L.lact_set_option(99, 1) == -1
    assert b"unknown option" in L.lact_last_error()
