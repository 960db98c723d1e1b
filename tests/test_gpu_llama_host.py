"""The reference's own host stack drives the HIP backend: oracle/_ref/llama_host (this repo's driver, linked against the
reference's llama.cpp layer and cactus layer compiled where they lie) loads libggml-hip.so with lm_ggml_backend_load(), then
goes through cactus_init_context_c -> cactus_context::loadModel -> common_init_from_params -> llama_model_load_from_file
(the load-time supports_op probes of cactus/llama-model.cpp:161-165,246-251, the buffer-type selection of :277-362, the
upload loop of cactus/llama-model-loader.cpp:913-1064), llama_decode, cactus_bench_c (cactus/cactus_bench.cpp:10-159)
and cactus_completion_c.  The model is a small random-init LLaMA-shaped GGUF that the driver writes with the reference's
gguf writer and weight quantizers (Q4_K / Q6_K mixed the way a Q4_K_M file mixes them).

What is compared: the logits of 53 positions (a 40-token prompt batch, three single-token steps, batches of 7 and 3)
with the backend against the same binary without it.

Tolerance.  Each matmul on its own meets the per-op tolerance (the graph tests feed both backends the same inputs).  End
to end the two runs drift apart more than that, and would between any two implementations that differ in the last bit:
an activation that lands within rounding distance of a Q8_K step quantizes to the neighbouring integer, which turns a
1e-7 relative difference into one quantization step (max|x| / 127) on that element.  Measured per node on this model the
normalized mean squared error goes 4e-14 (layer-0 Q) -> 6e-8 (layer-0 attention output) -> 1.4e-5 (layer-0 FFN output)
-> 3e-4 at the logits, roughly NMSE_out = 0.01 * sqrt(NMSE_in) per quantized matmul, which has its fixed point near
1e-4..1e-3.  Position 0 attends to itself only and sees none of the other rows' flips: it stays at 1e-13.  The bounds
below are set from that: position 0 tight, everything else 2e-3, and the arg-max token must agree on 90 % of positions.
"""
import os
import subprocess

import numpy as np
import pytest

import cactus_amd

HERE = os.path.dirname(os.path.abspath(__file__))
HOST = os.path.join(HERE, "..", "oracle", "_ref", "llama_host")
N_VOCAB, ROWS = 4096, 53


def run_host(args, env_extra=None, timeout=300):
    if not os.path.exists(HOST):
        pytest.fail("oracle/_ref/llama_host is not built: run `make -C oracle host` where the reference tree is present")
    env = dict(os.environ)
    env.update(env_extra or {})
    p = subprocess.run([HOST] + args, capture_output=True, text=True, errors="replace", timeout=timeout, env=env)
    stats = {}
    for line in p.stdout.splitlines():
        f = line.split()
        if len(f) == 3 and f[0] == "stat":
            stats[f[1]] = int(f[2])
    return p, stats


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("llama_host") / "random_llama_q4_k_m.gguf")
    p, _ = run_host(["make-gguf", path])
    assert p.returncode == 0, p.stdout + p.stderr
    return path


@pytest.fixture(scope="module")
def cpu_logits(model, tmp_path_factory):
    out = str(tmp_path_factory.mktemp("llama_host_cpu") / "cpu.bin")
    p, stats = run_host(["run", model, out])
    assert p.returncode == 0, p.stdout + p.stderr
    assert stats["bench_ok"] == 1 and stats["completion_ok"] == 1
    y = np.fromfile(out, np.float32).reshape(ROWS, N_VOCAB)
    assert np.isfinite(y).all()
    return y


def test_host_runs_without_backend(cpu_logits):
    """The driver, the GGUF it writes and the reference stack work on their own (no GPU needed)."""
    assert 0.5 < cpu_logits.std() < 2.0


def nmse(a, b):
    return float(((a - b) ** 2).sum() / (a ** 2).sum())


@pytest.mark.gpu
@pytest.mark.parametrize("device_type,n_gpu_layers,use_mmap", [("ACCEL", 0, 0), ("GPU", 99, 0), ("GPU", 99, 1), ("GPU", 2, 0)])
def test_llama_decode_through_the_real_host(model, cpu_logits, tmp_path, device_type, n_gpu_layers, use_mmap):
    out = str(tmp_path / "hip.bin")
    p, stats = run_host(["run", model, out, cactus_amd.BACKEND_LIB, str(n_gpu_layers), str(use_mmap)],
                        {"CACTUS_HIP_DEVICE_TYPE": device_type, "LLAMA_HOST_VERBOSE": "1"})
    print(p.stdout[-3000:])
    assert p.returncode == 0, p.stdout[-4000:] + p.stderr[-4000:]
    assert "loaded HIP backend" in p.stderr
    assert stats["backend_devices"] == 1
    assert stats["bench_ok"] == 1 and stats["completion_ok"] == 1
    assert stats["mul_mat_nodes"] > 0
    # where the weights went: every tensor when the device is an accelerator or all layers are offloaded
    # (token_embd stays with the CPU for a GPU-type device: llama-model.cpp keeps the input layer there)
    if device_type == "ACCEL":
        assert stats["tensors_elsewhere"] == 0
    elif n_gpu_layers >= 5:
        assert stats["tensors_in_hip_buffers"] >= 38
    else:
        assert 0 < stats["tensors_in_hip_buffers"] < 38
    if use_mmap == 0:
        # llama-model-loader.cpp:913-984 chose the pinned staging buffers + events + set_tensor_async branch
        assert "using async uploads for device HIP0" in p.stderr
        assert stats["async_uploaded_bytes"] > 0
    else:
        assert stats["async_uploaded_bytes"] == 0 and stats["uploaded_bytes"] > 0
    y = np.fromfile(out, np.float32).reshape(ROWS, N_VOCAB)
    assert np.isfinite(y).all()
    per_row = [nmse(cpu_logits[r], y[r]) for r in range(ROWS)]
    agree = float(np.mean(cpu_logits.argmax(1) == y.argmax(1)))
    print(f"{device_type} ngl={n_gpu_layers} mmap={use_mmap}: NMSE position 0 {per_row[0]:.2e}, worst {max(per_row):.2e}, "
          f"all {nmse(cpu_logits, y):.2e}, arg-max agreement {agree:.3f}")
    assert per_row[0] < 1e-9
    assert max(per_row) < 2e-3
    assert agree >= 0.9
