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
