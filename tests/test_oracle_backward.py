"""Pins the backward stages of the oracle: bit-exact against the reference's own softmax_grad and
multiheadmatmulTN compiled into oracle/_ref (dense-causal special case), against the committed golden
fixture written from that build, and against torch autograd of a dense float64 attention for every
pattern; the TN look-up table against a brute-force column scan."""
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle_lib as orc
from test_oracle_attention import PATTERNS, causal_case, needs_ref, ref_dense_causal

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
P = orc._p


def ref_dense_causal_backward(Q, K, V, dO, scale):
    """The reference's dense CPU backward of the attention block (dV = P^T dO, dP = dO V^T,
    dS = softmax_grad, dK = dS^T Q, dQ = dS K) through its own functions."""
    B, L, H, d = Q.shape
    _, _, Pm = ref_dense_causal(Q, K, V, scale)
    t = lambda x: np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3)))
    qt, kt, vt, dot = t(Q), t(K), t(V), t(dO)
    dVt = np.zeros((B, H, L, d), np.float32)
    orc.ref.ref_multiheadmatmulTN(P(dVt), P(Pm), P(dot), B, H, L, L, d)
    dP = np.zeros((B, H, L, L), np.float32)
    orc.ref.ref_multiheadmatmulNT(P(dP), P(dot), P(vt), B, H, L, d, L)   # zero above the diagonal (matmul.h:65-73)
    dS = np.zeros_like(dP)
    orc.ref.ref_softmax_grad(P(dS), P(dP), P(Pm), ctypes.c_float(scale), B, H, L)
    dKt = np.zeros((B, H, L, d), np.float32)
    orc.ref.ref_multiheadmatmulTN(P(dKt), P(dS), P(qt), B, H, L, L, d)
    dQt = np.zeros((B, H, L, d), np.float32)
    orc.ref.ref_multiheadmatmulNN(P(dQt), P(dS), P(kt), B, H, L, L, d)
    return t(dQt), t(dKt), t(dVt), dS


@needs_ref
@pytest.mark.parametrize("bs,L,d", [(32, 128, 16), (64, 128, 64)])
def test_backward_bit_exact_vs_reference_dense_causal(bs, L, d):
    B, H = 2, 2
    scale = 1.0 / np.sqrt(d)
    Q, K, V, luts, words = causal_case(B, H, L, d, bs, seed=31)
    dO = orc.fill_normal((B, L, H, d), 35)
    want_dQ, want_dK, want_dV, dS_ref = ref_dense_causal_backward(Q, K, V, dO, scale)
    dQ, dK, dV, _ = orc.attention_backward(Q, K, V, dO, luts, bs, scale, mask=words)
    for got, want in ((dQ, want_dQ), (dK, want_dK), (dV, want_dV)):
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fixture", ["attention_backward_dense_causal.npz", "attention_dense_causal_block64.npz"])
def test_backward_matches_golden_fixture(fixture):
    fx = np.load(os.path.join(GOLDEN, fixture))
    B, L, H, d = (int(v) for v in fx["shape"])
    bs = int(fx["bs"])
    Q, K, V, luts, words = causal_case(B, H, L, d, bs, seed=int(fx["seed"]))
    dO = orc.fill_normal((B, L, H, d), int(fx["seed"]) + 4)
    assert np.array_equal(dO, fx["dO"])
    dQ, dK, dV, _ = orc.attention_backward(Q, K, V, dO, luts, bs, float(fx["scale"]), mask=words)
    for got, name in ((dQ, "dQ"), (dK, "dK"), (dV, "dV")):
        assert np.array_equal(got.view(np.uint32), fx[name].view(np.uint32))


@pytest.mark.parametrize("pattern", sorted(PATTERNS))
def test_backward_vs_torch_autograd_float64(pattern):
    bs, nb, B, H, d = 32, 6, 1, 2, 16
    L = bs * nb
    scale = 0.3
    layout = PATTERNS[pattern](nb)
    luts = orc.build_luts(layout)
    keep_blocks = (np.random.default_rng(3).random((luts["blocks"], bs, bs)) < 0.85).astype(np.uint8)
    words = orc.pack_mask(keep_blocks)
    valid = np.array([L - 20], np.int32)
    Q, K, V, dO = (orc.fill_normal((B, L, H, d), 50 + i) for i in range(4))
    dQ, dK, dV, _ = orc.attention_backward(Q, K, V, dO, luts, bs, scale, mask=words, valid_len=valid)
    keep = orc.dense_keep_matrix(layout, bs, keep_blocks=keep_blocks, nt_lut=luts["nt_lut"], valid=int(valid[0]))
    q, k, v = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (Q, K, V))
    s = torch.einsum("bihd,bjhd->bhij", q, k)
    m = torch.tensor(keep, dtype=torch.bool)[None, None]
    neg = torch.finfo(torch.float64).min
    smax = torch.where(m, s, torch.full_like(s, neg)).amax(-1, keepdim=True)
    e = torch.where(m, torch.exp((s - smax) * scale), torch.zeros_like(s))
    p = e / (e.sum(-1, keepdim=True) + 1e-6)
    o = torch.einsum("bhij,bjhd->bihd", p, v)
    o.backward(torch.tensor(dO, dtype=torch.float64))
    for got, want in ((dQ, q.grad), (dK, k.grad), (dV, v.grad)):
        want = want.numpy()
        assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("pattern", sorted(PATTERNS))
def test_tn_lut_is_the_column_scan(pattern):
    nb = 12
    layout = PATTERNS[pattern](nb)
    luts = orc.build_luts(layout)
    tn, tn_max = orc.build_tn_lut(luts["nt_lut"], nb)
    nt = luts["nt_lut"]
    at = nb
    for c in range(nb):
        rows = [r for r in range(nb) if layout[r, c]]
        assert tn[c, 0] == at and tn[c, 1] == len(rows)
        for r in rows:
            blk = int(tn[at, 0])
            assert tn[at, 1] == r and tuple(nt[blk]) == (r, c)
            at += 1
    assert at == nb + luts["blocks"] and tn_max == max(int(layout[:, c].sum()) for c in range(nb))
    # causal layout: the count pattern of the reference's commented builder (ewops.h:675-701): nb, nb-1, ..., 1
    causal = orc.build_luts(orc.layout_full(10, causal=True))
    tnc, mx = orc.build_tn_lut(causal["nt_lut"], 10)
    assert [int(x) for x in tnc[:10, 1]] == list(range(10, 0, -1)) and mx == 10 and int(tnc[0, 0]) == 10
