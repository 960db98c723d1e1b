"""chip_mul_mat_noalloc: the entry point that allocates nothing (its workspace is a static device array inside the
library) against chip_mul_mat with a caller workspace of the same size, bit for bit, through the C-ABI.

Two calls in a row share the array, the second on a smaller input: stale bytes of the first call (quantized rows of more
tokens, split-K partial tiles) must not reach the second result."""
import numpy as np
import pytest

import common
import oracle as O

pytestmark = pytest.mark.gpu


def run_pair(dev, wt, W, x, noalloc):
    """One mul_mat through the C-ABI; noalloc picks the entry point.  Returns y [n, N]."""
    L = dev.lib
    x = np.ascontiguousarray(x, np.float32)
    n, K = x.shape
    N = W.shape[0]
    nb01 = dev.row_size(wt, K)
    dW, dx, dy = dev.to_device(W), dev.to_device(x), dev.alloc(n * N * 4)
    dev.check(L.chip_memset(dy.ptr, 0xFF, n * N * 4, None))
    if noalloc:
        dev.check(L.chip_mul_mat_noalloc(wt, dW.ptr, nb01, K, N, dx.ptr, K, n, dy.ptr, N, None))
    else:
        wsz = L.chip_mul_mat_noalloc_max_workspace()
        ws = dev.alloc(wsz)
        dev.check(L.chip_memset(ws.ptr, 0xA5, wsz, None))
        dev.check(L.chip_mul_mat(wt, dW.ptr, nb01, K, N, dx.ptr, K, n, dy.ptr, N, ws.ptr, wsz, None))
    dev.sync()
    return dy.download(np.float32, n * N).reshape(n, N)


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q8_0, O.Q6_K, O.Q4_0), ids=lambda t: O.TYPE_NAMES[t])
def test_noalloc_equals_mul_mat_two_calls_in_a_row(orc, wt):
    import cactus_amd
    dev = cactus_amd.Device(0)
    assert dev.lib.chip_mul_mat_noalloc_max_workspace() == 16 << 20
    K, N = 4096, 300
    W = orc.quantize_weights(wt, common.weights_f32(90 + wt, N, K))
    # first call: 64 tokens on a matrix with few row tiles - the GEMM with K split (partial tiles in the array);
    # second call: 3 tokens on fewer rows - the GEMV over prepared rows, in the same array
    for n, rows in ((64, N), (3, 77), (1, N), (130, 200), (8, 31)):
        x = common.activations_f32(91 + n, n, K)
        got = run_pair(dev, wt, W[:rows], x, True)
        want = run_pair(dev, wt, W[:rows], x, False)
        assert got.tobytes() == want.tobytes(), (O.TYPE_NAMES[wt], n, rows)
        ref = orc.mul_mat(wt, W[:rows], x, nthreads=8, want=("sum_abs",))
        err = np.abs(got.astype(np.float64) - ref["y"].astype(np.float64))
        assert (err <= 1e-5 * ref["sum_abs"]).all(), (O.TYPE_NAMES[wt], n, rows)


def test_noalloc_leaves_device_memory_alone_and_replays_from_a_graph(orc):
    """After chip_init() and one warm call per shape (the first launch of a kernel raises its LDS limit, a host call), a
    call changes nothing about the device's free memory, and a call recorded under stream capture replays - three times,
    with other work and synchronizations in between - to the bits chip_mul_mat gives."""
    import ctypes as C
    import cactus_amd
    dev = cactus_amd.Device(0)
    L = dev.lib
    hip = C.CDLL("libamdhip64.so")
    K, N = 4096, 300
    wt = O.Q4_K
    W = orc.quantize_weights(wt, common.weights_f32(190, N, K))
    nb01 = dev.row_size(wt, K)
    dW = dev.to_device(W)
    st = C.c_void_p()
    dev.check(L.chip_stream_create(C.byref(st)))
    for n in (1, 8, 64):
        x = common.activations_f32(191 + n, n, K)
        want = run_pair(dev, wt, W, x, False)
        dx, dy = dev.to_device(x), dev.alloc(n * N * 4)
        dev.check(L.chip_mul_mat_noalloc(wt, dW.ptr, nb01, K, N, dx.ptr, K, n, dy.ptr, N, st))     # warm call
        dev.sync(st)
        free0, free1, tot = C.c_size_t(), C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free0), C.byref(tot)) == 0
        dev.check(L.chip_mul_mat_noalloc(wt, dW.ptr, nb01, K, N, dx.ptr, K, n, dy.ptr, N, st))
        dev.sync(st)
        assert hip.hipMemGetInfo(C.byref(free1), C.byref(tot)) == 0
        assert free0.value == free1.value, "the call changed the device's free memory"
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(st, 0) == 0
        rc = L.chip_mul_mat_noalloc(wt, dW.ptr, nb01, K, N, dx.ptr, K, n, dy.ptr, N, st)
        assert hip.hipStreamEndCapture(st, C.byref(graph)) == 0 and rc == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for rep in range(3):
            dev.check(L.chip_memset(dy.ptr, 0xFF, n * N * 4, st))
            dev.sync(st)
            assert hip.hipGraphLaunch(gexec, st) == 0
            dev.sync(st)
            got = dy.download(np.float32, n * N).reshape(n, N)
            assert got.tobytes() == want.tobytes(), (n, rep)
            run_pair(dev, wt, W[:50], common.activations_f32(5 + rep, 3, K), True)        # other work on the shared array
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)


def test_noalloc_rejects_what_does_not_fit():
    import cactus_amd
    dev = cactus_amd.Device(0)
    L = dev.lib
    K, N = 4096, 8
    n_big = 1 + (16 << 20) // L.chip_mul_mat_workspace_size(O.Q4_K, K, 1)
    buf = dev.alloc(1 << 16)
    assert L.chip_mul_mat_workspace_size(O.Q4_K, K, n_big) > L.chip_mul_mat_noalloc_max_workspace()
    # the size check comes before anything touches the pointers
    assert L.chip_mul_mat_noalloc(O.Q4_K, buf.ptr, dev.row_size(O.Q4_K, K), K, N, buf.ptr, K, n_big, buf.ptr, N, None) == -3
    assert L.chip_mul_mat_noalloc(O.Q4_K, buf.ptr, dev.row_size(O.Q4_K, K), 100, N, buf.ptr, K, 1, buf.ptr, N, None) == -2
    assert L.chip_mul_mat_noalloc(O.Q4_K, None, dev.row_size(O.Q4_K, K), K, N, buf.ptr, K, 1, buf.ptr, N, None) == -1
    assert L.chip_mul_mat_noalloc(O.Q4_K, buf.ptr, dev.row_size(O.Q4_K, K), K, 0, buf.ptr, K, 1, buf.ptr, N, None) == 0
    dev.sync()
