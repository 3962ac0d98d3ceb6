"""Parity of the unfused trio (sdd -> masked softmax -> dsd) and of the two-stage fusion
(sdd+softmax -> P) against the CPU oracle, through the C ABI."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, qkv, rel_err, run_fused
from sfb import sfb

pytestmark = pytest.mark.gpu
THREADS = 16


def setup(pattern, bs, nb, B, H, seed, bf16, masked=True):
    L, d = nb * bs, 64
    luts = sfb.build_luts(PATTERNS[pattern](nb))
    kind = {"causal": sfb.MASK_CAUSAL_DIAG, "local_causal": sfb.MASK_LOCAL}.get(pattern, sfb.MASK_ALL)
    mask = None
    if masked:
        if kind:
            mask = sfb.pack_mask(sfb.element_mask(luts["nt_lut"], bs, kind, local_attn_ctx=bs))
        else:
            keep = (np.random.default_rng(seed).random((luts["blocks"], bs, bs)) < 0.75).astype(np.uint8)
            mask = sfb.pack_mask(keep)
    Q, K, V = qkv(B, L, H, d, seed=seed, bf16=bf16)
    valid = np.array([L] + [L - bs - 3] * (B - 1), np.int32)
    return luts, mask, Q, K, V, valid


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("pattern", ["causal", "bigbird"])
def test_trio_stage_by_stage(pattern, bs, bf16):
    nb, B, H = 8, 2, 3
    luts, mask, Q, K, V, valid = setup(pattern, bs, nb, B, H, 7 + bs, bf16)
    tol = TOL_BF16 if bf16 else TOL_F32
    store = sfb.BF16 if bf16 else sfb.F32   # S and P storage type, as the configuration's precision
    blocks = luts["blocks"]
    nt, nn = sfb.to_device(luts["nt_lut"]), sfb.to_device(luts["nn_lut"])
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    S_want = orc.sdd_nt(Q, K, luts["nt_lut"], bs)
    P_want = orc.masked_softmax(S_want, luts["nn_lut"], nb, 0.125, mask=mask, valid_len=valid)
    O_want = orc.dsd_nn(P_want, V, luts["nn_lut"])

    S = sfb.bst_sgemm_nt(nt, q, k, bs, blocks, out_dtype=store)
    assert rel_err(S.float().cpu().numpy(), S_want) <= tol
    mask_rm = None if mask is None else sfb.to_device(sfb.transpose_mask(mask, blocks, bs))
    vl = sfb.to_device(valid)
    # softmax on the oracle's scores isolates this stage
    S_in = torch.from_numpy(S_want).cuda().to(S.dtype)
    P = sfb.BlocksparseMaskedSoftmax(nn, mask_rm, S_in, nb, 0.125, valid_len=vl, max_lut=luts["nn_max"])
    P_ref = orc.masked_softmax(S_in.float().cpu().numpy(), luts["nn_lut"], nb, 0.125, mask=mask, valid_len=valid)
    assert rel_err(P.float().cpu().numpy(), P_ref) <= tol
    masked_zero = (P_ref == 0)
    assert (P.float().cpu().numpy()[masked_zero] == 0).all()
    P_in = torch.from_numpy(P_want).cuda().to(S.dtype)
    magic, shift = sfb.magicu64(1)
    O = sfb.bst_sgemm_xn(nn, P_in, v, nb, op=sfb.NN_OP, magic=magic, shift=shift, max_lut=luts["nn_max"])
    O_ref = orc.dsd_nn(P_in.float().cpu().numpy(), V, luts["nn_lut"])
    assert rel_err(O.cpu().numpy(), O_ref) <= tol
    # the chain end to end, and against the fused kernel
    P2 = sfb.BlocksparseMaskedSoftmax(nn, mask_rm, S, nb, 0.125, valid_len=vl)
    O2 = sfb.bst_sgemm_xn(nn, P2, v, nb).cpu().numpy()
    assert rel_err(O2, O_want) <= (2 * tol if bf16 else tol)
    fused = run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16, mask=mask, valid_len=valid)
    assert rel_err(fused, O2) <= (2 * tol if bf16 else tol)


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("bf16", [False, True])
def test_fusion_attention2_probabilities(bs, bf16):
    nb, B, H = 8, 2, 3
    luts, mask, Q, K, V, valid = setup("bigbird", bs, nb, B, H, 31, bf16)
    S_want = orc.sdd_nt(Q, K, luts["nt_lut"], bs)
    P_want = orc.masked_softmax(S_want, luts["nn_lut"], nb, 0.125, mask=mask, valid_len=valid)
    q, k = dev(Q, bf16), dev(K, bf16)
    for out_dtype, tol in ((sfb.F32, TOL_BF16 if bf16 else TOL_F32), (sfb.BF16, TOL_BF16)):
        P = sfb.fusion_attention2(sfb.to_device(luts["nn_lut"]), q, k, bs, luts["blocks"], 0.125,
                                  mask=sfb.to_device(mask), valid_len=sfb.to_device(valid), out_dtype=out_dtype)
        got = P.float().cpu().numpy()
        assert rel_err(got, P_want) <= tol
        assert (got[P_want == 0] == 0).all()
    # rows sum to sum/(sum + 1e-6)
    rows = np.zeros((B, H, nb, bs))
    for blk, (r, _) in enumerate(luts["nt_lut"]):
        rows[:, :, r] += got[:, :, blk].sum(-1)
    assert np.abs(rows[0] - 1).max() < 2e-2


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("pattern", ["causal", "bigbird", "strided"])
def test_split_variant_with_flags_matches_the_row_owner_kernel(pattern, bs, bf16):
    """One work-group per block with flag / spin exchange (the reference's fusion_nt_softmax2 decomposition):
    same probabilities as the oracle and as fusion_attention2, status word zero."""
    nb, B, H = 16, 2, 3
    luts, mask, Q, K, V, valid = setup(pattern, bs, nb, B, H, 50 + bs, bf16)
    S = orc.sdd_nt(Q, K, luts["nt_lut"], bs)
    P_want = orc.masked_softmax(S, luts["nn_lut"], nb, 0.125, mask=mask, valid_len=valid)
    q, k = dev(Q, bf16), dev(K, bf16)
    nt, nn = sfb.to_device(luts["nt_lut"]), sfb.to_device(luts["nn_lut"])
    m, vl = (None if mask is None else sfb.to_device(mask)), sfb.to_device(valid)
    for _ in range(2):   # the second call finds used scratch: the call clears what it needs
        P, status = sfb.fusion_attention2_split(nt, nn, q, k, bs, luts["blocks"], 0.125, mask=m, valid_len=vl)
        torch.cuda.synchronize()
        assert int(status) == 0
        got = P.cpu().numpy()
        assert rel_err(got, P_want) <= (TOL_BF16 if bf16 else TOL_F32)
        assert (got[P_want == 0] == 0).all()
    row_owner = sfb.fusion_attention2(nn, q, k, bs, luts["blocks"], 0.125, mask=m, valid_len=vl)
    assert rel_err(got, row_owner.cpu().numpy()) <= 1e-5
    ordered = sfb.fusion_attention2(nn, q, k, bs, luts["blocks"], 0.125, mask=m, valid_len=vl,
                                    row_order=sfb.to_device(luts["row_order"]))
    assert torch.equal(ordered, row_owner)   # the order of the work does not change a bit of the result


def test_split_variant_gives_up_instead_of_waiting_forever():
    """With no polls allowed, a block whose block-row partners have not all arrived leaves without writing and
    reports it; every work-group still exits."""
    bs, nb, B, H = 64, 8, 1, 2
    luts, mask, Q, K, V, valid = setup("causal", bs, nb, B, H, 60, False, masked=False)
    q, k = dev(Q), dev(K)
    P, status = sfb.fusion_attention2_split(sfb.to_device(luts["nt_lut"]), sfb.to_device(luts["nn_lut"]), q, k, bs,
                                            luts["blocks"], 0.125, spin_limit=0)
    torch.cuda.synchronize()
    assert int(status) == 1


def test_c2_shape_unfused_chain_fp32():
    B, H, L, d, bs = 2, 12, 1024, 64, 32
    luts = sfb.build_luts(PATTERNS["fixed"](L // bs))
    Q, K, V = qkv(B, L, H, d, seed=2)
    valid = np.array([1000, 768], np.int32)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, valid_len=valid, nthreads=THREADS)
    q, k, v = (dev(x) for x in (Q, K, V))
    nn = sfb.to_device(luts["nn_lut"])
    S = sfb.bst_sgemm_nt(sfb.to_device(luts["nt_lut"]), q, k, bs, luts["blocks"])
    P = sfb.BlocksparseMaskedSoftmax(nn, None, S, L // bs, 0.125, valid_len=sfb.to_device(valid))
    O = sfb.bst_sgemm_xn(nn, P, v, L // bs).cpu().numpy()
    assert rel_err(O, want) <= TOL_F32


def test_empty_block_rows_give_zero_output():
    bs, nb, B, H = 32, 6, 1, 2
    lay = PATTERNS["local"](nb).copy()
    lay[4] = 0
    luts = sfb.build_luts(lay)
    Q, K, V = qkv(B, nb * bs, H, 64, seed=3)
    q, k, v = (dev(x) for x in (Q, K, V))
    nn = sfb.to_device(luts["nn_lut"])
    S = sfb.bst_sgemm_nt(sfb.to_device(luts["nt_lut"]), q, k, bs, luts["blocks"])
    P = sfb.BlocksparseMaskedSoftmax(nn, None, S, nb, 0.125)
    O = torch.full((B, nb * bs, H, 64), 7.0, device="cuda")
    sfb.bst_sgemm_xn(nn, P, v, nb, c=O)
    O = O.cpu().numpy()
    assert (O[:, 4 * bs:5 * bs] == 0).all()
    assert rel_err(O, orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125)) <= TOL_F32


@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("nb", [12, 24, 48, 70])
def test_softmax_every_rows_per_wave_variant(nb, bf16, masked):
    """Row lengths that select each register variant of the softmax kernel (4, 2 or 1 rows of a wave at a time,
    and the three-pass form), with causal rows so that one launch mixes them."""
    bs, B, H = 64, 2, 1
    luts = sfb.build_luts(sfb.layout_full(nb, causal=True))
    blocks = luts["blocks"]
    S = orc.fill_normal((B, H, blocks, bs, bs), 17)
    if bf16:
        S = orc.round_bf16(S)
    mask = valid = None
    if masked:
        mask = sfb.pack_mask(sfb.element_mask(luts["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG))
        valid = np.array([nb * bs, nb * bs - 70], np.int32)
    want = orc.masked_softmax(S, luts["nn_lut"], nb, 0.125, mask=mask, valid_len=valid)
    x = torch.from_numpy(S).cuda()
    got = sfb.BlocksparseMaskedSoftmax(
        sfb.to_device(luts["nn_lut"]), None if mask is None else sfb.to_device(sfb.transpose_mask(mask, blocks, bs)),
        x.to(torch.bfloat16) if bf16 else x, nb, 0.125, valid_len=None if valid is None else sfb.to_device(valid))
    got = got.float().cpu().numpy()
    assert rel_err(got, want) <= (TOL_BF16 if bf16 else TOL_F32)
    assert (got[want == 0] == 0).all()


@pytest.mark.parametrize("out_f32", [False, True])
def test_bf16_trio_per_head_tables_and_masks(out_f32):
    """The bf16 kernels for blocks of 64 with one look-up table and one mask per head: a block count that is not a
    multiple of the sdd's group of blocks, 9 (batch, head) pairs (not a multiple of the 8 XCDs), row lengths from
    1 to 19 blocks (register slots of the softmax, a row shared by the four waves, product rows that end inside a
    group of prefetched blocks), key padding, and both storage types for S and P."""
    bs, nb, B, H, d = 64, 19, 3, 3, 64
    L = nb * bs
    rng = np.random.default_rng(5)
    lays = []
    for h in range(H):
        lay = np.tril(np.ones((nb, nb), np.uint32))
        lays.append(np.roll(lay, h, axis=1) if h else lay)   # same number of blocks, other columns
    per_head = [sfb.build_luts(l) for l in lays]
    blocks = per_head[0]["blocks"]
    assert all(l["blocks"] == blocks for l in per_head) and blocks % 8 != 0
    nt = np.concatenate([l["nt_lut"] for l in per_head])
    nn = np.concatenate([l["nn_lut"] for l in per_head])
    keep = (rng.random((H, blocks, bs, bs)) < 0.8).astype(np.uint8)
    keep[:, :, :, 0] = 1
    mask = np.concatenate([sfb.pack_mask(keep[h]) for h in range(H)])
    mask_rows = np.concatenate([sfb.transpose_mask(sfb.pack_mask(keep[h]), blocks, bs) for h in range(H)])
    valid = np.array([L, L - 70, L - 5 * bs], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=21, bf16=True)
    store = sfb.F32 if out_f32 else sfb.BF16
    S = sfb.bst_sgemm_nt(sfb.to_device(nt), dev(Q, True), dev(K, True), bs, blocks, out_dtype=store, lut_heads=H)
    want_s = orc.sdd_nt(Q, K, nt, bs, lut_heads=H)
    assert rel_err(S.float().cpu().numpy(), want_s) <= TOL_BF16
    s_in = orc.round_bf16(want_s)
    want_p = orc.masked_softmax(s_in, nn, nb, 0.125, mask=mask, valid_len=valid, lut_heads=H, mask_heads=H)
    got_p = sfb.BlocksparseMaskedSoftmax(sfb.to_device(nn), sfb.to_device(mask_rows),
                                         torch.from_numpy(s_in).cuda().to(torch.bfloat16), nb, 0.125, out_dtype=store,
                                         valid_len=sfb.to_device(valid), lut_heads=H, mask_heads=H)
    got_p = got_p.float().cpu().numpy()
    assert rel_err(got_p, want_p) <= TOL_BF16
    assert (got_p[want_p == 0] == 0).all()
    p_in = orc.round_bf16(want_p)
    O = sfb.bst_sgemm_xn(sfb.to_device(nn), torch.from_numpy(p_in).cuda().to(torch.bfloat16), dev(V, True), nb,
                         lut_heads=H)
    assert rel_err(O.cpu().numpy(), orc.dsd_nn(p_in, V, nn, lut_heads=H)) <= TOL_BF16


def test_error_codes_instead_of_silent_no_op():
    q = torch.zeros((1, 64, 1, 64), device="cuda")
    lut = sfb.to_device(np.zeros((3, 2), np.uint32))
    p = lambda t: C.c_void_p(t.data_ptr())
    u = C.c_uint32
    # the reference silently ignores block sizes other than 32 (openai_blocksparse.h:225-232)
    assert sfb.lib.sfb_sdd_nt(None, p(lut), p(q), p(q), p(q), 0, 0, u(16), u(1), u(1), u(1), u(1), u(1), u(64),
                              u(1), u(1)) == 2
    assert sfb.lib.sfb_dsd_xn(None, p(lut), p(q), p(q), p(q), 0, 0, u(64), u(1), u(1), u(1), u(1), u(1), u(64),
                              u(1), u(2), u(sfb.NT_OP), u(1), u(0), u(1)) == 8
    assert sfb.lib.sfb_masked_softmax(None, p(lut), None, p(q), p(q), 0, 3, None, u(64), u(1), u(1), u(1), u(1),
                                      u(1), u(2), u(1), u(1), C.c_float(0.125)) == 5
    assert sfb.lib.sfb_fused_sdd_softmax(None, None, p(q), p(q), p(q), 0, 0, None, None, None, u(64), u(1), u(1), u(1),
                                         u(1), u(64), u(1), u(2), u(1), C.c_float(0.125)) == 1


@pytest.mark.needs_device
def test_cpp_host_program_through_reference_named_launchers():
    """sf-bert_amd/host/attention_host_test: a C++ main in the shape of the reference's *_fusion_test.cu
    that calls bst_sgemm_nt / BlocksparseMaskedSoftmax / bst_sgemm_xn / fusion_attention2 / fusion_attention."""
    import os
    import subprocess
    from sfb import ROOT
    exe = os.path.join(ROOT, "sf-bert_amd", "host", "attention_host_test")
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and "PASSED" in out.stdout
