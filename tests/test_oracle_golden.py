"""The oracle against the committed golden vectors (written by tests/golden/make_golden.py from the reference's
own compiled code).  Integer / byte outputs bit-exact; floats bit-exact too, because the oracle restates the
AVX2 accumulation order."""
import os

import numpy as np
import pytest

import oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def gold(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_mul_mat_golden(orc, wt):
    g = gold("mul_mat_%s.npz" % O.TYPE_NAMES[wt])
    K = int(g["K"])
    assert int(g["wtype"]) == wt
    # weight quantizer bytes (IQ4_NL's quantizer is not restated: its golden bytes come from the reference build)
    if wt in O.ORACLE_QUANTIZED:
        assert np.array_equal(orc.quantize_weights(wt, g["w"]), g["wq"])
    # dequantizer closed form
    assert np.array_equal(orc.dequantize(wt, g["wq"], K), g["w_deq"])
    # on-the-fly activation quantizer bytes
    at = O.VEC_DOT_TYPE[wt]
    assert np.array_equal(orc.quantize_activation(at, g["x"]), g["xq"])
    # dots and the whole op
    n, N = g["y_dot"].shape
    for t in range(n):
        for i in range(N):
            v = orc.vec_dot(wt, K, g["wq"][i], g["xq"][t])
            assert v.tobytes() == g["y_dot"][t, i].tobytes()
    out = orc.mul_mat(wt, g["wq"], g["x"], nthreads=2, want=("wdata", "sum_abs"))
    assert np.array_equal(out["y"], g["y_graph"])
    assert np.array_equal(out["wdata"], g["xq"])
    assert np.array_equal(g["y_graph"], g["y_dot"])      # MUL_MAT == n*N independent vec_dots
    assert (out["sum_abs"] > 0).all()


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q8_0), ids=lambda t: O.TYPE_NAMES[t])
def test_mul_mat_id_golden(orc, wt):
    g = gold("mul_mat_id_%s.npz" % O.TYPE_NAMES[wt])
    assert int(g["wtype"]) == wt
    out = orc.mul_mat_id(wt, g["W"], g["x"], g["ids"], nthreads=2)
    assert np.array_equal(out["y"], g["y_graph"])
    with pytest.raises(ValueError):                          # the reference asserts on ids outside [0, n_as)
        orc.mul_mat_id(wt, g["W"], g["x"], g["ids"] + 3)


def test_quantize_q8_0_edges(orc):
    g = gold("quantize_q8_0_edges.npz")
    with np.errstate(all="ignore"):
        got = orc.quantize_activation(O.Q8_0, g["x"])
        got_ref = np.stack([orc.quantize_q8_0_ref(r) for r in g["x"]])
    assert np.array_equal(got, g["q_avx2"])
    assert np.array_equal(got_ref, g["q_ref"])
    # the two quantizers really do differ on the tie rows (to-even vs away-from-zero): the fixture pins which
    assert not np.array_equal(g["q_avx2"][1], g["q_ref"][1])


def test_quantize_q8_1_edges(orc):
    g = gold("quantize_q8_1_edges.npz")
    with np.errstate(all="ignore"):
        got = orc.quantize_activation(O.Q8_1, g["x"])
    assert np.array_equal(got, g["q"])
    # same quants and d as Q8_0 on the same rows
    g0 = gold("quantize_q8_0_edges.npz")
    b1 = g["q"].reshape(g["q"].shape[0], -1, 36)
    b0 = g0["q_avx2"].reshape(g0["q_avx2"].shape[0], -1, 34)
    assert np.array_equal(b1[..., 4:], b0[..., 2:]) and np.array_equal(b1[..., :2], b0[..., :2])


def test_quantize_q8_K_edges(orc):
    g = gold("quantize_q8_K_edges.npz")
    got = orc.quantize_activation(O.Q8_K, g["x"])
    assert np.array_equal(got, g["q"])
    # sign rule: first largest element decides; row 1 has -2 first -> iscale > 0 -> +2 maps to +127
    q1 = got[1][4:260].view(np.int8)
    assert q1[3] == -127 and q1[7] == 127
    q2 = got[2][4:260].view(np.int8)
    assert q2[3] == -127 and q2[7] == 127   # +2 first -> iscale < 0 -> +2 maps to -127, -2 to +127
