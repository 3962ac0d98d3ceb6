"""Pins the oracle's whole-model pieces: the cross-entropy loss bit-exact against the reference's
softmax_cross_entropy_with_logits + to_one_hot (oracle/_ref) and the golden fixture written from it, and against
a float64 log-sum-exp; the transposed GEMM, the pre-LN layer and the model forward against float64 numpy."""
import ctypes
import os

import numpy as np
import pytest

import oracle_lib as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(orc.ref is None, reason="oracle/_ref not built (no reference checkout)")
P = orc._p


def test_cross_entropy_matches_golden_fixture():
    fx = np.load(os.path.join(GOLDEN, "softmax_cross_entropy.npz"))
    loss, rows, grad = orc.softmax_cross_entropy(fx["logits"], fx["labels"], want_grad=True)
    assert np.float32(loss).view(np.uint32) == fx["loss"].view(np.uint32)
    assert np.array_equal(grad.view(np.uint32), fx["grad"].view(np.uint32))


@needs_ref
@pytest.mark.parametrize("rows,vocab", [(8, 256), (6, 1000)])
def test_cross_entropy_bit_exact_vs_reference(rows, vocab):
    logits = orc.fill_normal((rows, vocab), 3) * 3
    labels = orc.fill_uniform_int((rows,), 4, 0, vocab - 1)
    d_ref, work, scratch = np.zeros_like(logits), logits.copy(), np.zeros((rows, vocab), np.int32)
    orc.ref.ref_softmax_cross_entropy.restype = ctypes.c_float
    want = np.float32(orc.ref.ref_softmax_cross_entropy(P(d_ref), P(work), P(labels), P(scratch), 2, rows // 2, vocab))
    loss, _, grad = orc.softmax_cross_entropy(logits, labels, want_grad=True)
    assert loss.view(np.uint32) == want.view(np.uint32)
    assert np.array_equal(grad.view(np.uint32), d_ref.view(np.uint32))


def test_cross_entropy_is_the_textbook_loss():
    rows, vocab = 40, 777
    logits = orc.fill_normal((rows, vocab), 5) * 4
    labels = orc.fill_uniform_int((rows,), 6, 0, vocab - 1)
    loss, row_loss, grad = orc.softmax_cross_entropy(logits, labels, want_grad=True)
    x = logits.astype(np.float64)
    lse = np.log(np.exp(x - x.max(1, keepdims=True)).sum(1)) + x.max(1)
    want_rows = lse - x[np.arange(rows), labels]
    assert np.abs(row_loss - want_rows).max() <= 1e-5 * np.abs(want_rows).max()
    assert abs(loss - want_rows.mean()) <= 1e-5 * want_rows.mean()
    sm = np.exp(x - lse[:, None])
    sm[np.arange(rows), labels] -= 1
    assert np.abs(grad - sm).max() <= 5e-6
    # a wrong label column or a missing 1/rows shows up immediately
    assert abs(loss - (lse - x[np.arange(rows), (labels + 1) % vocab]).mean()) > 1e-2


def test_sgemm_nt_is_a_textbook_product():
    A = orc.fill_normal((37, 96), 7)
    W = orc.fill_normal((53, 96), 8)
    want = A.astype(np.float64) @ W.astype(np.float64).T
    assert np.abs(orc.sgemm_nt(A, W, nthreads=2) - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(orc.sgemm_nt(A, W), orc.sgemm_nt(A, W, nthreads=3))


def make_model(n_layers, n, ffn, vocab, L, seed, tok_std=0.5):
    layers = []
    for i in range(n_layers):
        s = seed + 100 * i
        w = {}
        for j, (name, shape) in enumerate((("wq", (n, n)), ("wk", (n, n)), ("wv", (n, n)), ("wo", (n, n)),
                                           ("w1", (n, ffn)), ("w2", (ffn, n)))):
            w[name] = orc.fill_normal(shape, s + j, 0.08)
        for j, (name, size) in enumerate((("bq", n), ("bk", n), ("bv", n), ("bo", n), ("b1", ffn), ("b2", n))):
            w[name] = orc.fill_normal((size,), s + 10 + j, 0.1)
        w["ln1_g"] = orc.fill_normal((n,), s + 20, 0.1) + 1
        w["ln1_b"] = orc.fill_normal((n,), s + 21, 0.1)
        w["ln2_g"] = orc.fill_normal((n,), s + 22, 0.1) + 1
        w["ln2_b"] = orc.fill_normal((n,), s + 23, 0.1)
        layers.append(w)
    tok = orc.fill_normal((vocab, n), seed + 50, tok_std)
    pos = orc.fill_normal((L, n), seed + 51, 0.5)
    return layers, tok, pos


def f64_layer(x, w, keep, B, L, H, d, pre_ln):
    """float64 restatement of one layer; keep [L, L] bool."""
    w = {k: v.astype(np.float64) for k, v in w.items()}
    n = H * d

    def ln(t, g, b):
        mu = t.mean(-1, keepdims=True)
        var = (t * t).mean(-1, keepdims=True) - mu * mu
        return (t - mu) / np.sqrt(var + 1e-5) * g + b

    def attn(a):
        q = (a @ w["wq"] + w["bq"]).reshape(B, L, H, d)
        k = (a @ w["wk"] + w["bk"]).reshape(B, L, H, d)
        v = (a @ w["wv"] + w["bv"]).reshape(B, L, H, d)
        s = np.einsum("bqhd,bkhd->bhqk", q, k) / np.sqrt(d)
        s = np.where(keep[None, None], s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        return np.einsum("bhqk,bkhd->bqhd", p, v).reshape(B * L, n)

    gelu = lambda t: t / (1 + np.exp(-1.702 * t))
    if pre_ln:
        x1 = x + attn(ln(x, w["ln1_g"], w["ln1_b"])) @ w["wo"] + w["bo"]
        return x1 + gelu(ln(x1, w["ln2_g"], w["ln2_b"]) @ w["w1"] + w["b1"]) @ w["w2"] + w["b2"]
    x1 = ln(x + attn(x) @ w["wo"] + w["bo"], w["ln1_g"], w["ln1_b"])
    return ln(x1 + gelu(x1 @ w["w1"] + w["b1"]) @ w["w2"] + w["b2"], w["ln2_g"], w["ln2_b"])


@pytest.mark.parametrize("pre_ln", [True, False])
def test_model_forward_matches_float64(pre_ln):
    B, L, H, d, ffn, bs, vocab, n_layers = 2, 128, 2, 64, 256, 32, 61, 2
    n = H * d
    layout = orc.layout_local(L // bs, 1)
    luts = orc.build_luts(layout)
    keep_blocks = orc.element_mask(luts["nt_lut"], bs, 1)
    mask = orc.pack_mask(keep_blocks)
    layers, tok, pos = make_model(n_layers, n, ffn, vocab, L, seed=400)
    ids = orc.fill_uniform_int((B, L), 401, 0, vocab - 1)
    labels = orc.fill_uniform_int((B * L,), 402, 0, vocab - 1)
    loss, logits, hidden = orc.model_forward(ids, labels, tok, pos, layers, luts["nn_lut"], B, L, H, d, ffn, bs,
                                             luts["blocks"], pre_ln=pre_ln, mask=mask, nthreads=4)
    keep = orc.dense_keep_matrix(layout, bs, keep_blocks, luts["nt_lut"])
    x = (tok[ids] + pos[None]).astype(np.float64).reshape(B * L, n)
    for w in layers:
        x = f64_layer(x, w, keep, B, L, H, d, pre_ln)
    assert np.abs(hidden - x).max() <= 2e-5 * np.abs(x).max()
    lg = x @ tok.astype(np.float64).T
    assert np.abs(logits - lg).max() <= 2e-5 * np.abs(lg).max()
    lse = np.log(np.exp(lg - lg.max(1, keepdims=True)).sum(1)) + lg.max(1)
    want = (lse - lg[np.arange(B * L), labels]).mean()
    assert abs(loss - want) <= 1e-5 * want
    # the other wiring gives a visibly different result: the flag is not ignored
    other, _, _ = orc.model_forward(ids, labels, tok, pos, layers, luts["nn_lut"], B, L, H, d, ffn, bs,
                                    luts["blocks"], pre_ln=not pre_ln, mask=mask, nthreads=4)
    assert abs(other - loss) > 1e-3
