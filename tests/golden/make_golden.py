"""Writes tests/golden/*.npz from the reference's own compiled code (oracle/_ref/libggml_ref.so).

Run in the build container, where the reference tree is mounted:  python tests/golden/make_golden.py [type names]
(with type names, e.g. "q3_K q2_K", only the mul_mat fixtures of those types are written).
The fixtures hold data only: seeded inputs and the bytes / floats the reference produced for them.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle as O            # noqa: E402
import common                 # noqa: E402


def main():
    O.build()
    r = O.Reference()
    K, N, n = 512, 3, 2
    only = sys.argv[1:]
    for wt in O.WEIGHT_TYPES:
        name = O.TYPE_NAMES[wt]
        if only and name not in only:
            continue
        w = common.weights_f32(100 + wt, N, K, outliers=(wt in (O.Q4_K, O.Q6_K)))
        x = common.activations_f32(100 + wt, n, K)
        wq = r.quantize_weights(wt, w)
        at = O.VEC_DOT_TYPE[wt]
        xq = r.quantize_activation(at, x)
        y_dot = np.zeros((n, N), np.float32)
        for t in range(n):
            for i in range(N):
                y_dot[t, i] = r.vec_dot(wt, K, wq[i], xq[t])
        y_graph, _ = r.mul_mat_graph(wt, wq, x, nthreads=2)
        np.savez_compressed(os.path.join(HERE, "mul_mat_%s.npz" % name),
                            wtype=np.int32(wt), K=np.int32(K), w=w, x=x, wq=wq, xq=xq,
                            w_deq=r.dequantize(wt, wq, K), y_dot=y_dot, y_graph=y_graph)
    if only:
        return
    # LM_GGML_OP_MUL_MAT_ID from the reference's CPU graph: 5 experts, 3 used per token, per-slot activations for one
    # type and activations shared by a token's slots for the other
    for wt, ne11 in ((O.Q4_K, 1), (O.Q8_0, 3)):
        K, N, n_as, n_used, n_tokens = 512, 5, 5, 3, 3
        rng = np.random.default_rng(200 + wt)
        W = np.stack([r.quantize_weights(wt, common.weights_f32(200 + wt + e, N, K)) for e in range(n_as)])
        x = common.activations_f32(200 + wt, n_tokens * ne11, K).reshape(n_tokens, ne11, K)
        ids = np.stack([rng.permutation(n_as)[:n_used] for _ in range(n_tokens)]).astype(np.int32)
        ids[1] = ids[1, 0]                                   # one token sends all its slots to the same expert
        np.savez_compressed(os.path.join(HERE, "mul_mat_id_%s.npz" % O.TYPE_NAMES[wt]), wtype=np.int32(wt), W=W, x=x,
                            ids=ids, y_graph=r.mul_mat_id_graph(wt, W, x, ids, nthreads=2))
    e0 = common.q8_0_edge_rows()
    with np.errstate(all="ignore"):
        np.savez_compressed(os.path.join(HERE, "quantize_q8_0_edges.npz"), x=e0,
                            q_avx2=r.quantize_activation(O.Q8_0, e0),
                            q_ref=np.stack([r.quantize_q8_0_ref(row) for row in e0]))
        np.savez_compressed(os.path.join(HERE, "quantize_q8_1_edges.npz"), x=e0, q=r.quantize_activation(O.Q8_1, e0))
        ek = common.q8_K_edge_rows()
        np.savez_compressed(os.path.join(HERE, "quantize_q8_K_edges.npz"), x=ek,
                            q=r.quantize_activation(O.Q8_K, ek))
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
