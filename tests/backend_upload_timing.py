"""Timing of the model loader's two upload branches against the HIP backend (reference llama-model-loader.cpp:905-1064),
256 MB each, with a host memmove standing for file->read_raw:
  * asynchronous: n pinned staging buffers with an event each, set_tensor_async per chunk (the loader uses 4 x 1 MB);
  * blocking: the whole tensor read into a pageable buffer, then set_tensor.
Also prints the rates with the host copy left out (what the device side alone sustains).  Not a test (pytest does not
collect it):    python tests/backend_upload_timing.py
"""
import ctypes as C
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import oracle as O
from ggml_host import Host

host = Host()
host.reg = host.load_hip()
L = host.L
dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
host_buft = L.lm_ggml_backend_dev_host_buffer_type(dev)
total = 256 << 20
ctx = host.context()
a = L.lm_ggml_new_tensor_1d(ctx, O.F32, total // 4)
buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
be = L.lm_ggml_backend_dev_init(dev, None)
src = np.random.default_rng(0).integers(0, 256, total, dtype=np.uint8)

for n_buffers, chunk in ((4, 1 << 20), (4, 4 << 20), (2, 16 << 20)):
    bufs = [L.lm_ggml_backend_buft_alloc_buffer(host_buft, chunk) for _ in range(n_buffers)]
    ptrs = [L.lm_ggml_backend_buffer_get_base(hb) for hb in bufs]
    events = [L.lm_ggml_backend_event_new(dev) for _ in range(n_buffers)]
    for copy in (True, False):
        for rep in range(3):
            t0 = time.perf_counter()
            done = idx = 0
            waited = issued = 0.0
            while done < total:
                size = min(chunk, total - done)
                t1 = time.perf_counter()
                L.lm_ggml_backend_event_synchronize(events[idx])
                t2 = time.perf_counter()
                if copy:
                    C.memmove(ptrs[idx], src[done:done + size].ctypes.data, size)
                t3 = time.perf_counter()
                L.lm_ggml_backend_tensor_set_async(be, a, ptrs[idx], done, size)
                L.lm_ggml_backend_event_record(events[idx], be)
                waited += t2 - t1
                issued += time.perf_counter() - t3
                done += size
                idx = (idx + 1) % n_buffers
            for ev in events:
                L.lm_ggml_backend_event_synchronize(ev)
            dt = time.perf_counter() - t0
        print(f"async, {n_buffers} x {chunk >> 20} MB pinned, host copy {'in' if copy else 'left out'}: {total / dt / 1e9:.1f} GB/s "
              f"(of {dt * 1e3:.1f} ms: {waited * 1e3:.1f} waiting for events, {issued * 1e3:.1f} in set_tensor_async + event_record)", flush=True)

tmp = np.empty(total, np.uint8)
for copy in (True, False):
    for rep in range(3):
        t0 = time.perf_counter()
        if copy:
            C.memmove(tmp.ctypes.data, src.ctypes.data, total)
        L.lm_ggml_backend_tensor_set(a, tmp.ctypes.data_as(C.c_void_p), 0, total)
        dt = time.perf_counter() - t0
    print(f"blocking set_tensor from pageable memory, host copy {'in' if copy else 'left out'}: {total / dt / 1e9:.1f} GB/s", flush=True)
