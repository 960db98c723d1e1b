"""Not a test (pytest does not collect it): the 8-token GEMV kernels, one weight type at a time on a 14336 x 4096 matrix
(the trace's ffn_gate / ffn_up shape), every launch on a different copy of the weights, issued eagerly so that
`rocprofv3 --kernel-trace --stats -- python3 tests/mmv_profile_cases.py` sees one kernel name per case.
profiles/matrix_core_gemv_batch8_kernel_stats.md is made from its output."""
import ctypes as C
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import bench
import cactus_amd as ca

N, K, n, CALLS = 14336, 4096, 8, 200
dev, hip = ca.Device(0), bench.Hip()
L = dev.lib
rng = np.random.default_rng(3)
st = C.c_void_p()
dev.check(L.chip_stream_create(C.byref(st)))
x = dev.to_device(rng.standard_normal((n, K)).astype(np.float32))
y = dev.alloc(n * N * 4)
for wt in (ca.Q8_0, ca.Q4_0, ca.Q4_K, ca.Q5_K, ca.Q6_K):
    m = bench.RotatingWeights(dev, wt, N, K, rng)
    wsz = L.chip_mul_mat_workspace_size_n(wt, K, N, n)
    ws = dev.alloc(wsz)
    dev.check(L.chip_mul_mat_prepare(wt, K, x.ptr, K, n, ws.ptr, wsz, st))
    e0, e1 = hip.event(), hip.event()
    for it in range(CALLS + 3):
        if it == 3:
            hip.record(e0, st)
        dev.check(L.chip_mul_mat_run_ws(wt, m.next(), m.nb01, K, N, n, ws.ptr, wsz, y.ptr, N, st))
    hip.record(e1, st)
    dev.sync(st)
    us = hip.elapsed_ms(e0, e1) * 1e3 / CALLS
    print("%s %dx%d, %d tokens over prepared rows: %.2f us per eager launch, weights %.1f MB -> %.0f GB/s"
          % (ca.TYPE_NAMES[wt], N, K, n, us, m.bytes / 1e6, m.bytes / us / 1e3), flush=True)
    m.buf.free()
    ws.free()
