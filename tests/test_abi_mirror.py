"""The ABI mirror header against the reference's own headers (compile-time check; needs the reference tree)."""
import os
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference/cactus"


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference tree not mounted")
def test_mirror_matches_reference_headers():
    with tempfile.TemporaryDirectory() as tmp:
        cmd = ["g++", "-std=gnu++17", "-fsyntax-only", "-DLM_GGML_COMMON_DECL_CPP", "-I", REF, "-I", os.path.join(ROOT, "include"),
               os.path.join(ROOT, "tests", "abi_mirror_check.cpp")]
        r = subprocess.run(cmd, capture_output=True, text=True, cwd=tmp)
        assert r.returncode == 0, r.stderr[-4000:]
