"""Pins the oracle's encoder-layer ops: bit-exact against the reference's CPU functions (oracle/_ref)
and the golden fixtures written from them; float64 numpy / torch for the textbook behaviour."""
import os

import numpy as np
import pytest
import torch

import oracle_lib as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(orc.ref is None, reason="oracle/_ref not built (no reference checkout)")
P = orc._p


def test_layer_ops_match_golden_fixture():
    fx = np.load(os.path.join(GOLDEN, "layer_ops.npz"))
    x, g, b = fx["x"], fx["g"], fx["b"]
    ln, mean, rstd = orc.layernorm(x, g, b)
    assert np.array_equal(ln, fx["layernorm"]) and np.array_equal(mean, fx["mean"])
    assert np.array_equal(rstd, fx["rstd"])
    assert np.array_equal(orc.gelu(x), fx["gelu"])
    assert np.array_equal(orc.bias(x, g), fx["bias"])


@needs_ref
def test_layer_ops_bit_exact_vs_reference():
    rows, state = 64, 768
    x = orc.fill_normal((rows, state), 5) * 2 - 0.3
    g = orc.fill_normal((state,), 6)
    b = orc.fill_normal((state,), 7)
    want, mean, rstd = np.zeros_like(x), np.zeros(rows, np.float32), np.zeros(rows, np.float32)
    orc.ref.ref_layernorm(P(want), P(mean), P(rstd), P(x), P(g), P(b), 4, 16, state)
    got, m2, r2 = orc.layernorm(x, g, b)
    assert np.array_equal(got, want) and np.array_equal(m2, mean) and np.array_equal(r2, rstd)
    want = np.zeros_like(x)
    orc.ref.ref_gelu(P(want), P(x), 4, 16, state)
    assert np.array_equal(orc.gelu(x), want)
    orc.ref.ref_bias(P(want), P(x), P(g), state, rows)
    assert np.array_equal(orc.bias(x, g), want)
    y = orc.fill_normal((rows, state), 8)
    orc.ref.ref_tensor_add_tensor(P(want), P(x), P(y), 4, 16, state)
    got = np.zeros_like(x)
    orc.lib.orc_add(P(got), P(x), P(y), orc.C.c_long(x.size))
    assert np.array_equal(got, want)
    pos = orc.fill_normal((16, state), 9)
    orc.ref.ref_tensor_add_matrix(P(want), P(x), P(pos), 4, 16, state)
    orc.lib.orc_add_matrix(P(got), P(x), P(pos), 4, orc.C.c_long(16 * state))
    assert np.array_equal(got, want)
    table = orc.fill_normal((100, state), 10)
    ids = orc.fill_uniform_int((rows,), 11, 0, 99)
    orc.ref.ref_embedding_lookup(P(want), P(table), P(ids), 4, 16, 12, 64)
    orc.lib.orc_embedding_lookup(P(got), P(table), P(ids), orc.C.c_long(rows), state)
    assert np.array_equal(got, want) and np.array_equal(got, table[ids])
    src = orc.fill_normal((2, 5, 3, 4), 12)
    want4, got4 = np.zeros((2, 3, 5, 4), np.float32), np.zeros((2, 3, 5, 4), np.float32)
    orc.ref.ref_transpose_0123to0213(P(src), P(want4), 2, 5, 3, 4)
    orc.lib.orc_transpose_0213(P(src), P(got4), 2, 5, 3, 4)
    assert np.array_equal(got4, want4) and np.array_equal(got4, src.transpose(0, 2, 1, 3))


def test_layer_ops_textbook():
    rows, state = 32, 768
    x = orc.fill_normal((rows, state), 21) * 1.5 + 0.2
    g = orc.fill_normal((state,), 22)
    b = orc.fill_normal((state,), 23)
    got, _, _ = orc.layernorm(x, g, b)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (state,),
                                          torch.from_numpy(g).double(), torch.from_numpy(b).double(),
                                          eps=1e-5).numpy()
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    x64 = x.astype(np.float64)
    assert np.abs(orc.gelu(x) - x64 / (1 + np.exp(-1.702 * x64))).max() <= 1e-6
    A = orc.fill_normal((17, 96), 24)
    W = orc.fill_normal((96, 40), 25)
    got = orc.sgemm(A, W, nthreads=2)
    want = A.astype(np.float64) @ W.astype(np.float64)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(got, orc.sgemm(A, W, nthreads=1))


def _layer_f64(x, w, keep, B, L, H, d, rnd):
    r = (lambda a: orc.round_bf16(a).astype(np.float64)) if rnd else (lambda a: a.astype(np.float64))
    ln = lambda t, g, b: ((t - t.mean(-1, keepdims=True)) /
                          np.sqrt(t.var(-1, keepdims=True) + 1e-5)) * g + b
    x64 = x.astype(np.float64)
    xr = r(x)
    q = (xr @ r(w["wq"]) + w["bq"]).reshape(B, L, H, d)
    k = (xr @ r(w["wk"]) + w["bk"]).reshape(B, L, H, d)
    v = (xr @ r(w["wv"]) + w["bv"]).reshape(B, L, H, d)
    q, k, v = (r(t.astype(np.float32)) for t in (q, k, v))
    a = orc.dense_attention_f64(q, k, v, keep, 1 / np.sqrt(d)).reshape(B * L, H * d)
    a = r(a.astype(np.float32))
    x1 = ln(x64 + a @ r(w["wo"]) + w["bo"], w["ln1_g"], w["ln1_b"])
    f = r(x1.astype(np.float32)) @ r(w["w1"]) + w["b1"]
    f = f / (1 + np.exp(-1.702 * f))
    f = r(f.astype(np.float32))
    return ln(x1 + f @ r(w["w2"]) + w["b2"], w["ln2_g"], w["ln2_b"])


@pytest.mark.parametrize("bf16", [False, True])
def test_encoder_layer_vs_float64(bf16):
    B, L, H, d, ffn, bs = 2, 256, 4, 16, 128, 32
    n = H * d
    nb = L // bs
    lay = orc.layout_bigbird(nb, 1, 2, True, orc.bigbird_draw(nb, 1, 2, True, 2, 3))
    luts = orc.build_luts(lay)
    w = {k: orc.fill_normal(s, 200 + i, 0.05) for i, (k, s) in enumerate(
        [("wq", (n, n)), ("wk", (n, n)), ("wv", (n, n)), ("wo", (n, n)), ("w1", (n, ffn)),
         ("w2", (ffn, n)), ("bq", (n,)), ("bk", (n,)), ("bv", (n,)), ("bo", (n,)), ("b1", (ffn,)),
         ("b2", (n,)), ("ln1_g", (n,)), ("ln1_b", (n,)), ("ln2_g", (n,)), ("ln2_b", (n,))])}
    w["ln1_g"] = w["ln1_g"] + 1
    w["ln2_g"] = w["ln2_g"] + 1
    x = orc.fill_normal((B * L, n), 300)
    got = orc.encoder_layer(x, w, luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"],
                            operands_bf16=bf16, nthreads=2)
    want = _layer_f64(x, w, orc.dense_keep_matrix(lay, bs), B, L, H, d, bf16)
    tol = 2e-3 if bf16 else 2e-5  # bf16: a rounding point may flip by one bf16 ulp between float and double
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
