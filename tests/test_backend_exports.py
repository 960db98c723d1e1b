"""CPU-only: libggml-hip.so exists and exports what include/ggml_backend_hip.h declares, and leaves exactly
the host's ggml helpers undefined."""
import os
import re
import subprocess

import cactus_amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_backend_library_symbols():
    hdr = open(os.path.join(ROOT, "include", "ggml_backend_hip.h")).read()
    declared = sorted(set(re.findall(r"CACTUS_GGML_API\s+[\w\s\*]+?\b(lm_ggml_\w+)\s*\(", hdr)))
    assert "lm_ggml_backend_init" in declared and "lm_ggml_backend_hip_reg" in declared
    out = subprocess.run(["nm", "-D", cactus_amd.BACKEND_LIB], capture_output=True, text=True, check=True).stdout
    defined = set(re.findall(r" T (\w+)", out))
    undefined = set(re.findall(r" U (\w+)", out))
    for name in declared:
        assert name in defined, name
    host_syms = {s for s in undefined if s.startswith("lm_ggml_")}
    assert host_syms == {"lm_ggml_backend_buffer_init", "lm_ggml_nbytes", "lm_ggml_log_internal"}
    assert {s for s in undefined if s.startswith("chip_")} <= set(cactus_amd.EXPORTS)
