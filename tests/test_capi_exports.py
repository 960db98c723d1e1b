"""CPU-only: the C-ABI library is present, loads, and exports every symbol include/cactus_hip.h declares.
No compute call is made (there is no GPU here)."""
import ctypes
import os
import re

import cactus_amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    return sorted(set(re.findall(r"CHIP_API\s+[\w\s\*]+?\b(chip_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols("cactus_hip.h") == sorted(cactus_amd.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(cactus_amd.KERNEL_LIB)
    for name in declared_symbols("cactus_hip.h"):
        assert hasattr(lib, name), name


def test_layout_queries_need_no_gpu():
    lib = cactus_amd.load_library()
    assert [lib.chip_block_bytes(t) for t in (2, 8, 12, 14, 15)] == [18, 34, 144, 210, 292]
    assert [lib.chip_block_bytes(t) for t in (6, 13, 20, 3, 7, 9)] == [22, 176, 18, 20, 24, 36]
    assert lib.chip_vec_dot_type(cactus_amd.Q4_1) == cactus_amd.Q8_1 and lib.chip_vec_dot_type(cactus_amd.Q5_K) == cactus_amd.Q8_K
    assert lib.chip_row_size(cactus_amd.Q4_0, 4096) == 2304
    assert lib.chip_row_size(cactus_amd.Q4_K, 4096) == 2304
    assert lib.chip_row_size(cactus_amd.Q6_K, 14336) == 11760
    assert lib.chip_vec_dot_type(cactus_amd.Q4_0) == cactus_amd.Q8_0
    assert lib.chip_vec_dot_type(cactus_amd.Q6_K) == cactus_amd.Q8_K
    assert lib.chip_mul_mat_supported(cactus_amd.Q4_K, 4096) == 1
    assert lib.chip_mul_mat_supported(cactus_amd.Q4_K, 4000) == 0
    assert lib.chip_mul_mat_supported(cactus_amd.F16, 4096) == 1 and lib.chip_vec_dot_type(cactus_amd.F16) == cactus_amd.F16
    assert lib.chip_mul_mat_supported(30, 4096) == 0          # BF16 weights are not on this path
    assert lib.chip_mul_mat_workspace_size(cactus_amd.Q8_0, 4096, 3) == 3 * (4096 + 12 * 128)   # qs, d, sum, s planes
    # Q8_K planes (qs, d, bsums) of K = 4096 take 4672 bytes; token strides are multiples of 128
    assert lib.chip_mul_mat_workspace_size(cactus_amd.Q4_K, 4096, 3) == 3 * 4736
    assert lib.chip_error_string(-2).decode().startswith("unsupported")


def test_gelu_table_is_the_reference_table():
    """chip_gelu_table runs on the host (no GPU): the 65536 fp16 entries equal the oracle's restatement of lm_ggml_cpu_init's
    loop (pinned on the reference build in test_oracle_vs_ref), NaN entries included."""
    import ctypes as C
    import numpy as np
    import cactus_amd
    import oracle as O
    lib = C.CDLL(cactus_amd.KERNEL_LIB)
    t = np.zeros(65536, np.uint16)
    assert lib.chip_gelu_table(t.ctypes.data_as(C.c_void_p)) == 0
    assert np.array_equal(t, O.Oracle().gelu_table())
    assert t[0x3c00] != 0 and t[0] == 0                                  # gelu(1) = 0.84, gelu(0) = 0
