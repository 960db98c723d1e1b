"""The workgroup -> tile map of the GEMM kernels, checked on the host: a bijection onto the tiles, balanced over the eight
XCDs, block-local.  The check program includes the kernels' own header, so it tests the code the kernels run."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")
def test_xcd_tile_map_is_a_balanced_bijection(tmp_path):
    exe = str(tmp_path / "tile_map_check")
    cmd = ["hipcc", "-O1", "-std=c++17", "--offload-arch=gfx950", "-I", os.path.join(ROOT, "cactus_amd", "csrc"),
           os.path.join(ROOT, "tests", "tile_map_check.hip"), "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    shapes = []
    for rt in (1, 2, 3, 7, 8, 9, 31, 32, 33, 56, 112, 224, 251, 448):
        for tt in (1, 2, 3, 4, 7, 8, 9, 16, 17, 32, 33, 100):
            for conc in (32, 64):
                shapes.append("%d %d %d" % (rt, tt, conc))
    r = subprocess.run([exe], input="\n".join(shapes) + "\n", capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip() == "ok %d" % len(shapes), r.stdout[-2000:] + r.stderr[-2000:]
