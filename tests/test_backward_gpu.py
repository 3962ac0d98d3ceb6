"""Parity of the backward stages of the unfused attention path (softmax gradient, transposed block-sparse
product) and of their composition against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, qkv, rel_err
from sfb import sfb

pytestmark = pytest.mark.gpu


def rounded(x, bf16):
    return orc.round_bf16(x) if bf16 else x


def sparse_dev(x, bf16):
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t.to(torch.bfloat16) if bf16 else t


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("pattern", ["causal", "bigbird", "local"])
def test_softmax_grad(pattern, bs, bf16):
    nb, B, H = 8, 2, 3
    luts = sfb.build_luts(PATTERNS[pattern](nb))
    blocks = luts["blocks"]
    S = orc.fill_normal((B, H, blocks, bs, bs), 3)
    keep = (np.random.default_rng(bs).random((blocks, bs, bs)) < 0.75).astype(np.uint8)
    P = rounded(orc.masked_softmax(S, luts["nn_lut"], nb, 0.125, mask=sfb.pack_mask(keep)), bf16)
    dP = rounded(orc.fill_normal((B, H, blocks, bs, bs), 4), bf16)
    want = orc.masked_softmax_grad(dP, P, luts["nn_lut"], nb, 0.125)
    got = sfb.BlocksparseMaskedSoftmaxGrad(sfb.to_device(luts["nn_lut"]), sparse_dev(dP, bf16), sparse_dev(P, bf16),
                                           nb, 0.125, max_lut=luts["nn_max"])
    got = got.float().cpu().numpy()
    assert rel_err(got, want) <= (TOL_BF16 if bf16 else TOL_F32)
    assert (got[P == 0] == 0).all()   # masked keys carry no gradient


@pytest.mark.parametrize("bs", [8, 16])
@pytest.mark.parametrize("bf16", [False, True])
def test_softmax_and_its_gradient_at_small_block_sizes(bs, bf16):
    """Block sizes 8 and 16 exist for the softmax stages only (blocksparse.h:703-720, 1199-1224): uint8 / uint16
    mask words, 64 / 32 key blocks per wave step; nb 80 gives rows of one and of several steps."""
    nb, B, H = 80, 2, 2
    luts = sfb.build_luts(sfb.layout_full(nb, causal=True))
    blocks = luts["blocks"]
    S = rounded(orc.fill_normal((B, H, blocks, bs, bs), 40), bf16)
    mask = sfb.pack_mask(sfb.element_mask(luts["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG))
    assert mask.dtype.itemsize == bs // 8
    valid = np.array([nb * bs, nb * bs - bs - 3], np.int32)
    want = orc.masked_softmax(S, luts["nn_lut"], nb, 0.125, mask=mask, valid_len=valid)
    nn = sfb.to_device(luts["nn_lut"])
    P = sfb.BlocksparseMaskedSoftmax(nn, sfb.to_device(sfb.transpose_mask(mask, blocks, bs)), sparse_dev(S, bf16), nb,
                                     0.125, valid_len=sfb.to_device(valid))
    tol = TOL_BF16 if bf16 else TOL_F32
    got = P.float().cpu().numpy()
    assert rel_err(got, want) <= tol and (got[want == 0] == 0).all()
    plain = sfb.BlocksparseMaskedSoftmax(nn, None, sparse_dev(S, bf16), nb, 0.125).float().cpu().numpy()
    assert rel_err(plain, orc.masked_softmax(S, luts["nn_lut"], nb, 0.125)) <= tol
    Pw = rounded(want, bf16)
    dP = rounded(orc.fill_normal((B, H, blocks, bs, bs), 41), bf16)
    dS = sfb.BlocksparseMaskedSoftmaxGrad(nn, sparse_dev(dP, bf16), sparse_dev(Pw, bf16), nb, 0.125)
    assert rel_err(dS.float().cpu().numpy(), orc.masked_softmax_grad(dP, Pw, luts["nn_lut"], nb, 0.125)) <= tol


@pytest.mark.parametrize("bs,nb", [(64, 70), (32, 132)])
def test_softmax_grad_rows_longer_than_the_register_cache(bs, nb):
    luts = sfb.build_luts(sfb.layout_full(nb, causal=False))
    blocks = luts["blocks"]
    S = orc.fill_normal((1, 1, blocks, bs, bs), 5)
    P = orc.masked_softmax(S, luts["nn_lut"], nb, 0.125)
    dP = orc.fill_normal((1, 1, blocks, bs, bs), 6)
    want = orc.masked_softmax_grad(dP, P, luts["nn_lut"], nb, 0.125)
    got = sfb.BlocksparseMaskedSoftmaxGrad(sfb.to_device(luts["nn_lut"]), sparse_dev(dP, False),
                                           sparse_dev(P, False), nb, 0.125)
    assert rel_err(got.cpu().numpy(), want) <= TOL_F32


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("nb", [12, 24, 48])
def test_softmax_grad_every_rows_per_wave_variant(nb, bf16):
    """Row lengths that select each register variant of the kernel (4, 2 or 1 rows of a wave at a time), with
    causal rows so that one launch mixes them."""
    bs = 64
    luts = sfb.build_luts(sfb.layout_full(nb, causal=True))
    blocks = luts["blocks"]
    S = orc.fill_normal((1, 2, blocks, bs, bs), 15)
    P = rounded(orc.masked_softmax(S, luts["nn_lut"], nb, 0.125), bf16)
    dP = rounded(orc.fill_normal((1, 2, blocks, bs, bs), 16), bf16)
    want = orc.masked_softmax_grad(dP, P, luts["nn_lut"], nb, 0.125)
    got = sfb.BlocksparseMaskedSoftmaxGrad(sfb.to_device(luts["nn_lut"]), sparse_dev(dP, bf16), sparse_dev(P, bf16),
                                           nb, 0.125)
    assert rel_err(got.float().cpu().numpy(), want) <= (TOL_BF16 if bf16 else TOL_F32)


def test_softmax_grad_in_place_and_per_head_luts():
    bs, nb, B, H = 64, 8, 2, 4
    lays = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lays[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    assert all(l["blocks"] == blocks for l in per_head)
    nn = np.concatenate([l["nn_lut"] for l in per_head])
    S = orc.fill_normal((B, H, blocks, bs, bs), 8)
    P = orc.masked_softmax(S, nn, nb, 0.125, lut_heads=H)
    dP = orc.fill_normal((B, H, blocks, bs, bs), 9)
    want = orc.masked_softmax_grad(dP, P, nn, nb, 0.125, lut_heads=H)
    buf = sparse_dev(dP, False)
    got = sfb.BlocksparseMaskedSoftmaxGrad(sfb.to_device(nn), buf, sparse_dev(P, False), nb, 0.125, lut_heads=H,
                                           dx=buf)
    assert got.data_ptr() == buf.data_ptr()
    assert rel_err(got.cpu().numpy(), want) <= TOL_F32


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("a_bf16,x_bf16", [(False, False), (True, True), (True, False), (False, True)])
@pytest.mark.parametrize("pattern", ["causal", "bigbird"])
def test_transposed_product(pattern, bs, a_bf16, x_bf16):
    nb, B, H, d = 8, 2, 3, 64
    lay = PATTERNS[pattern](nb).copy()
    lay[:, 5] = 0   # a key-block column without blocks: its output rows are zeros
    luts = sfb.build_luts(lay)
    blocks = luts["blocks"]
    A = rounded(orc.fill_normal((B, H, blocks, bs, bs), 11), a_bf16)
    X = rounded(orc.fill_normal((B, nb * bs, H, d), 12), x_bf16)
    want = orc.dsd_tn(A, X, luts["tn_lut"])
    out = torch.full((B, nb * bs, H, d), 7.0, device="cuda")
    magic, shift = sfb.magicu64(1)
    sfb.bst_sgemm_xn(sfb.to_device(luts["tn_lut"]), sparse_dev(A, a_bf16), dev(X, x_bf16), nb, op=sfb.TN_OP,
                     magic=magic, shift=shift, max_lut=luts["tn_max"], c=out)
    got = out.cpu().numpy()
    assert (got[:, 5 * bs:6 * bs] == 0).all()
    # the inputs are exact in both precisions and the sums are fp32 on both sides
    assert rel_err(got, want) <= TOL_F32


def test_transposed_product_per_head_luts_and_rectangular_result():
    bs, nb, B, H, d = 64, 8, 1, 4, 64
    lays = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lays[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    tn = np.concatenate([l["tn_lut"] for l in per_head])
    A = orc.round_bf16(orc.fill_normal((B, H, blocks, bs, bs), 13))
    X = orc.round_bf16(orc.fill_normal((B, nb * bs, H, d), 14))
    want = orc.dsd_tn(A, X, tn, lut_heads=H)
    got = sfb.bst_sgemm_xn(sfb.to_device(tn), sparse_dev(A, True), dev(X, True), nb, op=sfb.TN_OP, lut_heads=H)
    assert rel_err(got.cpu().numpy(), want) <= TOL_F32


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("pattern", ["causal", "bigbird", "strided"])
def test_attention_backward(pattern, bs, bf16):
    nb, B, H, d = 8, 2, 3, 64
    luts = sfb.build_luts(PATTERNS[pattern](nb))
    blocks = luts["blocks"]
    kind = sfb.MASK_CAUSAL_DIAG if pattern == "causal" else sfb.MASK_ALL
    mask = sfb.pack_mask(sfb.element_mask(luts["nt_lut"], bs, kind)) if kind else None
    Q, K, V = qkv(B, nb * bs, H, d, seed=21 + bs, bf16=bf16)
    dO = rounded(orc.fill_normal((B, nb * bs, H, d), 30), bf16)
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, 0.125, mask=mask)
    q, k, v, do = (dev(x, bf16) for x in (Q, K, V, dO))
    luts_dev = {name: sfb.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    # forward probabilities from the library's own forward (sdd + masked softmax), stored in the working precision
    p = sfb.fusion_attention2(luts_dev["nn_lut"], q, k, bs, blocks, 0.125,
                              mask=None if mask is None else sfb.to_device(mask),
                              out_dtype=sfb.BF16 if bf16 else sfb.F32)
    assert rel_err(p.float().cpu().numpy(), P) <= (TOL_BF16 if bf16 else TOL_F32)
    dq, dk, dv = sfb.attention_backward(q, k, v, do, p, luts_dev, bs, blocks, 0.125)
    tol = TOL_BF16 if bf16 else TOL_F32
    for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        assert rel_err(got.cpu().numpy(), want) <= tol, name
    # with the forward output: dP and the softmax gradient in one kernel, the row term taken from dO . O
    o = sfb.fused_attention(q, k, v, luts_dev["nn_lut"], bs, blocks, 0.125,
                            mask=None if mask is None else sfb.to_device(mask))
    delta = sfb.row_dot(do, o).cpu().numpy()
    want_delta = np.einsum("blhd,blhd->bhl", dO.astype(np.float64), orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125,
                                                                                    mask=mask).astype(np.float64))
    assert np.abs(delta - want_delta).max() <= tol * np.abs(want_delta).max()
    dq2, dk2, dv2 = sfb.attention_backward(q, k, v, do, p, luts_dev, bs, blocks, 0.125, o=o)
    for name, got, want in (("dq", dq2, dQ), ("dk", dk2, dK), ("dv", dv2, dV)):
        assert rel_err(got.cpu().numpy(), want) <= tol, name
    # the three dsd products launched over work items, block-rows and block-columns of more than 3 blocks cut
    schedules = sfb.dsd_schedules(luts, nb, B, H, bs, d, max_blocks=3)
    for forward_output in (None, o):
        dq3, dk3, dv3 = sfb.attention_backward(q, k, v, do, p, luts_dev, bs, blocks, 0.125, o=forward_output,
                                               schedules=schedules)
        for name, got, want in (("dq", dq3, dQ), ("dk", dk3, dK), ("dv", dv3, dV)):
            assert rel_err(got.cpu().numpy(), want) <= tol, name


@pytest.mark.parametrize("d", [32, 96, 128])
@pytest.mark.parametrize("bs,store_bf16", [(32, False), (64, False), (64, True)])
def test_unfused_forward_and_backward_at_other_head_sizes(d, bs, store_bf16):
    """fp32 Q/K/V/dO with head size 32, 96 or 128; S, P, dP, dS stored in fp32 or bf16: every product kernel
    (NT, NN, TN) and the two-stage fusion (its per-block comparison variant stays at head size 64)."""
    nb, B, H = 8, 2, 2
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    blocks = luts["blocks"]
    scale = float(1.0 / np.sqrt(d))
    Q, K, V = qkv(B, nb * bs, H, d, seed=3 * d + bs)
    dO = orc.fill_normal((B, nb * bs, H, d), 90 + d)
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, scale)
    q, k, v, do = (dev(x) for x in (Q, K, V, dO))
    ld = {name: sfb.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    code = sfb.BF16 if store_bf16 else sfb.F32
    tol = TOL_BF16 if store_bf16 else TOL_F32
    p = sfb.fusion_attention2(ld["nn_lut"], q, k, bs, blocks, scale, out_dtype=code)
    assert rel_err(p.float().cpu().numpy(), P) <= tol
    S = sfb.bst_sgemm_nt(ld["nt_lut"], q, k, bs, blocks, out_dtype=code)
    assert rel_err(S.float().cpu().numpy(), orc.sdd_nt(Q, K, luts["nt_lut"], bs)) <= tol
    O = sfb.bst_sgemm_xn(ld["nn_lut"], p, v, nb)
    assert rel_err(O.cpu().numpy(), orc.attention(Q, K, V, luts["nn_lut"], bs, scale)) <= tol
    dq, dk, dv = sfb.attention_backward(q, k, v, do, p, ld, bs, blocks, scale)
    for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        assert rel_err(got.cpu().numpy(), want) <= tol, name
    dq, dk, dv = sfb.attention_backward(q, k, v, do, p, ld, bs, blocks, scale, o=O)
    for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        assert rel_err(got.cpu().numpy(), want) <= tol, name


