"""Pins the oracle's arithmetic: bit-exact against the reference's own CPU functions compiled into
oracle/_ref (dense-causal special case), against the committed golden fixtures written from that
build, float64 brute force for every pattern, closed forms and torch SDPA."""
import os

import numpy as np
import pytest
import torch

import oracle_lib as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(orc.ref is None, reason="oracle/_ref not built (no reference checkout)")
P = orc._p


def causal_case(B, H, L, d, bs, seed):
    Q = orc.fill_normal((B, L, H, d), seed)
    K = orc.fill_normal((B, L, H, d), seed + 1)
    V = orc.fill_normal((B, L, H, d), seed + 2)
    luts = orc.build_luts(orc.layout_full(L // bs, causal=True))
    words = orc.pack_mask(orc.element_mask(luts["nt_lut"], bs, orc.MASK_CAUSAL_DIAG))
    return Q, K, V, luts, words


def ref_dense_causal(Q, K, V, scale):
    """transformer.cpp:533-545 through the reference's own functions."""
    B, L, H, d = Q.shape
    qt, kt, vt = (np.zeros((B, H, L, d), np.float32) for _ in range(3))
    for src, dst in ((Q, qt), (K, kt), (V, vt)):
        orc.ref.ref_transpose_0123to0213(P(np.ascontiguousarray(src)), P(dst), B, L, H, d)
    S = np.zeros((B, H, L, L), np.float32)
    orc.ref.ref_multiheadmatmulNT(P(S), P(qt), P(kt), B, H, L, d, L)
    Pm = np.zeros_like(S)
    import ctypes
    orc.ref.ref_softmax(P(Pm), P(S), ctypes.c_float(scale), L, B, H)
    Ot = np.zeros((B, H, L, d), np.float32)
    orc.ref.ref_multiheadmatmulNN(P(Ot), P(Pm), P(vt), B, H, L, L, d)
    O = np.zeros((B, L, H, d), np.float32)
    orc.ref.ref_transpose_0123to0213(P(Ot), P(O), B, H, L, d)
    return O, S, Pm


@needs_ref
@pytest.mark.parametrize("bs,L,d", [(32, 128, 16), (64, 128, 64), (32, 64, 8)])
def test_attention_bit_exact_vs_reference_dense_causal(bs, L, d):
    B, H = 2, 3
    scale = 1.0 / np.sqrt(d)
    Q, K, V, luts, words = causal_case(B, H, L, d, bs, seed=11)
    want, S_ref, P_ref = ref_dense_causal(Q, K, V, scale)
    got = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, mask=words)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the three stages separately reproduce the same bits
    S = orc.sdd_nt(Q, K, luts["nt_lut"], bs)
    Pm = orc.masked_softmax(S, luts["nn_lut"], L // bs, scale, mask=words)
    for blk, (r, c) in enumerate(luts["nt_lut"].tolist()):
        ref_blk = S_ref[:, :, r * bs:(r + 1) * bs, c * bs:(c + 1) * bs]
        keep = np.tril(np.ones((bs, bs), bool)) if r == c else np.ones((bs, bs), bool)
        assert np.array_equal(np.where(keep, S[:, :, blk], 0), ref_blk)
        assert np.array_equal(Pm[:, :, blk], P_ref[:, :, r * bs:(r + 1) * bs, c * bs:(c + 1) * bs])
    O3 = orc.dsd_nn(Pm, V, luts["nn_lut"])
    assert np.array_equal(O3, want)


@pytest.mark.parametrize("fixture", ["attention_dense_causal.npz", "attention_dense_causal_block64.npz"])
def test_attention_matches_golden_fixture(fixture):
    fx = np.load(os.path.join(GOLDEN, fixture))
    B, L, H, d = (int(v) for v in fx["shape"])
    bs = int(fx["bs"])
    Q, K, V, luts, words = causal_case(B, H, L, d, bs, seed=int(fx["seed"]))
    assert np.array_equal(Q, fx["Q"])
    got = orc.attention(Q, K, V, luts["nn_lut"], bs, float(fx["scale"]), mask=words)
    assert np.array_equal(got.view(np.uint32), fx["O"].view(np.uint32))


PATTERNS = {
    "local": lambda nb: orc.layout_local(nb, 1, bidirectional=True),
    "local_causal": lambda nb: orc.layout_local(nb, 1),
    "fixed": lambda nb: orc.layout_fixed(1, nb, 4, causal=False)[0],
    "strided": lambda nb: orc.layout_strided(nb, 4, 4),
    "bigbird": lambda nb: orc.layout_bigbird(nb, 1, 2, True, orc.bigbird_draw(nb, 1, 2, True, 3, 5)),
    "full": lambda nb: orc.layout_full(nb, causal=False),
}


@pytest.mark.parametrize("pattern", sorted(PATTERNS))
@pytest.mark.parametrize("bs", [32, 64])
def test_attention_vs_float64_brute_force(pattern, bs):
    nb, B, H, d = 8, 2, 2, 32
    L = nb * bs
    scale = 1.0 / np.sqrt(d)
    lay = PATTERNS[pattern](nb)
    luts = orc.build_luts(lay)
    Q, K, V = (orc.fill_normal((B, L, H, d), 100 + i) for i in range(3))
    kind = orc.MASK_LOCAL if pattern == "local_causal" else orc.MASK_ALL
    keep_blocks = orc.element_mask(luts["nt_lut"], bs, kind, local_attn_ctx=bs)
    words = orc.pack_mask(keep_blocks) if kind else None
    valid = np.array([L, L - bs - 7], np.int32)
    got = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, mask=words, valid_len=valid)
    keeps = [orc.dense_keep_matrix(lay, bs, keep_blocks, luts["nt_lut"], int(v)) for v in valid]
    want = orc.dense_attention_f64(Q, K, V, keeps, scale)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    # staged == fused, bit for bit
    S = orc.sdd_nt(Q, K, luts["nt_lut"], bs)
    Pm = orc.masked_softmax(S, luts["nn_lut"], nb, scale, mask=words, valid_len=valid)
    assert np.array_equal(orc.dsd_nn(Pm, V, luts["nn_lut"]), got)


def test_all_ones_closed_form_and_fully_masked_rows():
    # all-ones inputs (fixed_fusion_test.cu:263-268): S == d, P uniform over kept keys, O == sum/(sum+1e-6)
    bs, nb, B, H, d = 32, 4, 1, 2, 16
    L = bs * nb
    ones = np.ones((B, L, H, d), np.float32)
    lay = orc.layout_local(nb, 1, bidirectional=True)
    luts = orc.build_luts(lay)
    O = orc.attention(ones, ones, ones, luts["nn_lut"], bs, 0.25)
    n_keys = lay.sum(axis=1) * bs
    for r in range(nb):
        want = np.float32(n_keys[r]) / (np.float32(n_keys[r]) + np.float32(1e-6))
        assert np.allclose(O[0, r * bs:(r + 1) * bs], want, rtol=1e-6)
    # valid_len = 0 masks every key: sum = 0 -> 0/(1e-6) = exactly 0 (ewops.h:93)
    O0 = orc.attention(ones, ones, ones, luts["nn_lut"], bs, 0.25, valid_len=np.zeros(B, np.int32))
    assert (O0 == 0).all()
    # a block-row without blocks gives zeros as well
    lay2 = lay.copy()
    lay2[1] = 0
    O1 = orc.attention(ones, ones, ones, orc.build_luts(lay2)["nn_lut"], bs, 0.25)
    assert (O1[0, bs:2 * bs] == 0).all() and (O1[0, :bs] != 0).all()


def test_full_layout_equals_torch_sdpa():
    bs, nb, B, H, d = 32, 4, 2, 3, 64
    L = bs * nb
    Q, K, V = (orc.fill_normal((B, L, H, d), 7 + i) for i in range(3))
    luts = orc.build_luts(orc.layout_full(nb, causal=False))
    got = orc.attention(Q, K, V, luts["nn_lut"], bs, 1 / 8.0)
    t = lambda a: torch.from_numpy(a).double().permute(0, 2, 1, 3)
    want = torch.nn.functional.scaled_dot_product_attention(t(Q), t(K), t(V)).permute(0, 2, 1, 3).numpy()
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()


def test_key_block_permutation_invariance():
    # permuting the key blocks (and V with them) inside every row leaves O unchanged up to summation order
    bs, nb, B, H, d = 32, 6, 1, 2, 32
    L = bs * nb
    Q, K, V = (orc.fill_normal((B, L, H, d), 40 + i) for i in range(3))
    lay = orc.layout_full(nb, causal=False)
    luts = orc.build_luts(lay)
    perm = np.random.default_rng(3).permutation(nb)
    tok = (perm[:, None] * bs + np.arange(bs)[None]).reshape(-1)
    O1 = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.2)
    O2 = orc.attention(Q, K[:, tok].copy(), V[:, tok].copy(), luts["nn_lut"], bs, 0.2)
    assert np.abs(O1 - O2).max() <= 1e-5 * np.abs(O1).max()


def test_per_head_luts_and_masks():
    bs, nb, B, H, d = 32, 8, 1, 4, 16
    L = bs * nb
    lay = orc.layout_fixed(H, nb, 4, causal=True)
    per_head = [orc.build_luts(lay[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    assert all(p["blocks"] == blocks for p in per_head)
    nn = np.concatenate([p["nn_lut"] for p in per_head])
    masks = np.concatenate([orc.pack_mask(orc.element_mask(p["nt_lut"], bs, orc.MASK_CAUSAL_DIAG))
                            for p in per_head])
    Q, K, V = (orc.fill_normal((B, L, H, d), 60 + i) for i in range(3))
    got = orc.attention(Q, K, V, nn, bs, 0.25, mask=masks, lut_heads=H, mask_heads=H, blocks=blocks)
    for h in range(H):
        keep = orc.dense_keep_matrix(lay[h], bs, orc.element_mask(per_head[h]["nt_lut"], bs,
                                                                  orc.MASK_CAUSAL_DIAG),
                                     per_head[h]["nt_lut"])
        want = orc.dense_attention_f64(Q[:, :, h:h + 1], K[:, :, h:h + 1], V[:, :, h:h + 1], keep, 0.25)
        assert np.abs(got[:, :, h:h + 1] - want).max() <= 2e-5 * np.abs(want).max()
