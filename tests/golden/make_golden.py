"""Writes the golden fixtures in this directory by running the REFERENCE's own CPU functions (the
C++ headers of /root/reference compiled into oracle/_ref/libsfbert_ref.so by oracle/Makefile) on
small seeded inputs.  Run once where the reference checkout exists:  python tests/golden/make_golden.py
The fixtures hold inputs and expected outputs only."""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as orc  # noqa: E402
from test_oracle_attention import causal_case, ref_dense_causal  # noqa: E402

P = orc._p


def main():
    assert orc.ref is not None, "build oracle/_ref first (make -C oracle)"
    B, H, L, d, bs, seed = 1, 2, 128, 16, 32, 2024
    scale = np.float32(1.0 / np.sqrt(d))
    Q, K, V, _, _ = causal_case(B, H, L, d, bs, seed)
    O, _, _ = ref_dense_causal(Q, K, V, float(scale))
    np.savez_compressed(os.path.join(HERE, "attention_dense_causal.npz"), Q=Q, K=K, V=V, O=O,
                        shape=np.array([B, L, H, d]), bs=bs, seed=seed, scale=scale)

    from test_oracle_backward import ref_dense_causal_backward
    dO = orc.fill_normal((B, L, H, d), seed + 4)
    dQ, dK, dV, _ = ref_dense_causal_backward(Q, K, V, dO, float(scale))
    np.savez_compressed(os.path.join(HERE, "attention_backward_dense_causal.npz"), dO=dO, dQ=dQ, dK=dK, dV=dV,
                        shape=np.array([B, L, H, d]), bs=bs, seed=seed, scale=scale)

    # a second shape: blocks of 64, head size 64 (the benchmarked tile shape)
    B, H, L, d, bs, seed = 1, 1, 192, 64, 64, 2025
    scale = np.float32(1.0 / np.sqrt(d))
    Q, K, V, _, _ = causal_case(B, H, L, d, bs, seed)
    O, _, _ = ref_dense_causal(Q, K, V, float(scale))
    dO = orc.fill_normal((B, L, H, d), seed + 4)
    dQ, dK, dV, _ = ref_dense_causal_backward(Q, K, V, dO, float(scale))
    np.savez_compressed(os.path.join(HERE, "attention_dense_causal_block64.npz"), Q=Q, K=K, V=V, O=O, dO=dO, dQ=dQ, dK=dK,
                        dV=dV, shape=np.array([B, L, H, d]), bs=bs, seed=seed, scale=scale)

    rows, state = 6, 48
    x = orc.fill_normal((rows, state), 77) * 3 + 0.5
    g = orc.fill_normal((state,), 78)
    b = orc.fill_normal((state,), 79)
    ln, mean, rstd = (np.zeros_like(x), np.zeros(rows, np.float32), np.zeros(rows, np.float32))
    orc.ref.ref_layernorm(P(ln), P(mean), P(rstd), P(x), P(g), P(b), 2, 3, state)
    ge = np.zeros_like(x)
    orc.ref.ref_gelu(P(ge), P(x), 2, 3, state)
    bi = np.zeros_like(x)
    orc.ref.ref_bias(P(bi), P(x), P(g), state, rows)
    np.savez_compressed(os.path.join(HERE, "layer_ops.npz"), x=x, g=g, b=b, layernorm=ln, mean=mean,
                        rstd=rstd, gelu=ge, bias=bi)
    rows, vocab = 12, 50
    logits = orc.fill_normal((rows, vocab), 81) * 2
    labels = orc.fill_uniform_int((rows,), 82, 0, vocab - 1)
    d_out, work, scratch = np.zeros_like(logits), logits.copy(), np.zeros((rows, vocab), np.int32)
    orc.ref.ref_softmax_cross_entropy.restype = ctypes.c_float
    loss = orc.ref.ref_softmax_cross_entropy(P(d_out), P(work), P(labels), P(scratch), 3, 4, vocab)
    np.savez_compressed(os.path.join(HERE, "softmax_cross_entropy.npz"), logits=logits, labels=labels,
                        loss=np.float32(loss), grad=d_out)
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()
