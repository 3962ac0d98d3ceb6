"""GPU parity tests of the wider coverage: peaked bf16 rows and the error budget of the two bf16 loops, scheduled
launches with one table per head, head sizes that are not multiples of 32 (fused forward, unfused sequence, both
backward paths), the fused backward with fp32 tensors and the unfused path with bf16 tensors at head sizes
32 / 96 / 128.  Everything through the C ABI against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, qkv, rel_err, run_fused
from sfb import sfb
from test_full_size_gpu import per_head_errors, scheduled
from test_fused_attention_gpu import check
from test_fused_backward_gpu import forward

pytestmark = pytest.mark.gpu
THREADS = 16


def test_c4_error_budget_of_the_two_bf16_loops():
    """The benchmarked launch takes the loop that folds the scale into the score product (power-of-two part on the
    queries, which is exact, the rest in fp32 per score) and sums the unrounded probabilities; a launch with key
    padding -- here a valid length of the whole context, which masks nothing -- takes the loop that follows the
    running maximum.  Both against the oracle at the full size: the first must stay within half the tolerance and
    within 2.5 times the second's error."""
    B, H, L, d, bs = 4, 12, 4096, 64, 64
    luts = sfb.build_luts(PATTERNS["bigbird"](L // bs))
    max_blocks = sfb.suggest_max_blocks(luts["nn_lut"], L // bs, B * H)
    Q, K, V = qkv(B, L, H, d, seed=406, bf16=True)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    lean, sched = scheduled(Q, K, V, luts, bs, 0.125, True, max_blocks)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    general = sfb.fused_attention_scheduled(q, k, v, sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"]), sched,
                                            ws, bs, luts["blocks"], 0.125,
                                            valid_len=sfb.to_device(np.full(B, L, np.int32))).cpu().numpy()
    e_lean, e_general = per_head_errors(lean, want).max(), per_head_errors(general, want).max()
    print("lean loop %.3e, general loop %.3e" % (e_lean, e_general), flush=True)
    assert e_general <= 5e-3
    # (the arithmetic model in test_scale_split.py puts the two at 2.0-2.7e-3 and 1.4-1.6e-3)
    assert e_lean <= 5e-3 and e_lean <= 2.5 * e_general


@pytest.mark.parametrize("qmul,scale", [(6.0, 0.125), (1.0, 1.0), (2.0, 1.0), (6.0, 1.0)])
def test_large_scores_bf16(qmul, scale):
    """Peaked rows with bf16 tensors, through the scheduled and the streamed launch without mask: |score * scale| of
    30 to 90, exponents up to 2^85 above the offset of the row's first block, so the loop with the fixed offset is
    what runs (the last case passes 2^100 and is redone by the loop that follows the maximum).  The error must not
    grow with the scores: the scale's power-of-two part on the queries is exact and the rest is applied in fp32."""
    bs, nb, B, H, d = 64, 8, 2, 3, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    Q, K, V = qkv(B, L, H, d, seed=91)
    Q, K, V = orc.round_bf16(Q * qmul), orc.round_bf16(K), orc.round_bf16(V)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, scale)
    got = run_fused(Q, K, V, luts, bs, scale, bf16=True, max_blocks=4)
    err = rel_err(got, want)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    stream = sfb.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=16)
    ws = torch.zeros(sfb.stream_workspace_bytes(stream, d), dtype=torch.uint8, device="cuda")
    streamed = sfb.fused_attention_streamed(q, k, v, sfb.to_device(luts["nn_lut"]), sfb.to_device(stream["blob"]), stream,
                                            ws, bs, luts["blocks"], scale)
    torch.cuda.synchronize()
    err_streamed = rel_err(streamed.cpu().numpy(), want)
    print("scheduled %.3e, streamed %.3e" % (err, err_streamed), flush=True)
    assert sfb.stream_status(stream, d, ws) == 0
    assert err <= 0.75 * TOL_BF16 and err_streamed <= 0.75 * TOL_BF16


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("bs", [32, 64])
def test_scheduled_launch_with_per_head_tables(bf16, bs):
    """The reference's `fixed` pattern gives every head its own layout (fixed_fusion_test.cu:38-39, 58-106): the
    scheduled launch with one look-up table, one mask and one work-item list per head, rows cut in chunks of 2."""
    nb, B, H, d = 16, 3, 4, 64
    L = bs * nb
    lay = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lay[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    assert all(p["blocks"] == blocks for p in per_head)
    nn = np.concatenate([p["nn_lut"] for p in per_head])
    masks = np.concatenate([sfb.pack_mask(sfb.element_mask(p["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG)) for p in per_head])
    Q, K, V = qkv(B, L, H, d, seed=81, bf16=bf16)
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    tol = TOL_BF16 if bf16 else TOL_F32
    for max_blocks in (2, 100):
        sched = sfb.build_schedule_heads(nn, nb, H, max_blocks)
        assert (sched["n_parts"] > 0) == (max_blocks == 2)
        ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
        for mask in (masks, None):
            want = orc.attention(Q, K, V, nn, bs, 0.125, mask=mask, lut_heads=H, mask_heads=H if mask is not None else 1,
                                 blocks=blocks, nthreads=THREADS)
            outs = []
            for _ in range(2):   # the second launch finds the arrival counters as the first one left them
                out = torch.full((B, L, H, d), 7.0, device="cuda")
                sfb.fused_attention_scheduled_heads(q, k, v, sfb.to_device(nn), sfb.to_device(sched["items"]), sched, ws,
                                                    bs, blocks, 0.125, mask=None if mask is None else sfb.to_device(mask),
                                                    mask_heads=H if mask is not None else 1, out=out)
                torch.cuda.synchronize()
                outs.append(out.cpu().numpy())
            assert np.array_equal(outs[0], outs[1])
            diff = np.abs(outs[0].astype(np.float64) - want).max(axis=(0, 1, 3)) / np.abs(want).max()
            print("max_blocks", max_blocks, "masked", mask is not None, "error per head", diff, flush=True)
            assert diff.max() <= tol


@pytest.mark.parametrize("d,bf16", [(16, True), (48, True), (80, True), (112, True), (40, True), (8, True), (120, True),
                                    (16, False), (48, False), (80, False), (112, False), (36, False), (4, False),
                                    (100, False)])
@pytest.mark.parametrize("bs", [32, 64])
def test_head_sizes_that_are_not_multiples_of_32(d, bs, bf16):
    """The reference's K64 = false kernels take any head size that is a multiple of 4 (openai_blocksparse.h:221-222).
    Here: multiples of 4 (fp32) or 8 (bf16 -- rows of whole 16-byte vectors) up to 128, through the kernel of the
    next multiple of 32 with zero-padded queries; plain, scheduled and streamed launches, with and without mask and
    padding, a row without blocks, split rows merged from partial records, bf16 output, log-sum-exp output."""
    nb, B, H = 8, 2, 3
    L = nb * bs
    tol = TOL_BF16 if bf16 else TOL_F32
    lay = PATTERNS["bigbird"](nb)
    lay[5] = 0
    luts = sfb.build_luts(lay)
    keep = (np.random.default_rng(d).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    mask = sfb.pack_mask(keep)
    valid = np.array([L, L - bs - 5], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=3 * d + bs, bf16=bf16)
    scale = float(1.0 / np.sqrt(d))
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, mask=mask, valid_len=valid, nthreads=THREADS)
    plain = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, nthreads=THREADS)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16, mask=mask, valid_len=valid), want, tol)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16, mask=mask, valid_len=valid, max_blocks=3), want, tol)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16), plain, tol)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16, max_blocks=3), plain, tol)
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    sched = sfb.build_schedule(luts["nn_lut"], nb, 3)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    nn, items = sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"])
    if d % 8 == 0:
        o16 = sfb.fused_attention_scheduled(q, k, v, nn, items, sched, ws, bs, luts["blocks"], scale, out_dtype=sfb.BF16)
        torch.cuda.synchronize()
        assert rel_err(o16.float().cpu().numpy(), plain) <= max(tol, 2.0 ** -7)
    o32, lse = sfb.fused_attention_forward_lse(q, k, v, nn, items, sched, ws, bs, luts["blocks"], scale)
    torch.cuda.synchronize()
    check(o32.cpu().numpy(), plain, tol)
    assert torch.isfinite(lse).all() and float(lse[:, :, 5 * bs:6 * bs].abs().max()) == 0.0
    # streamed launches: rows cut into chunks, merged from partial records
    stream = sfb.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=64)
    assert stream["plan"].n_parts > 0
    sws = torch.zeros(sfb.stream_workspace_bytes(stream, d), dtype=torch.uint8, device="cuda")
    blob = sfb.to_device(stream["blob"])
    for m, vl, ref in ((None, None, plain), (sfb.to_device(mask), sfb.to_device(valid), want)):
        for _ in range(2):   # the second launch finds the flags as the first one left them
            out = sfb.fused_attention_streamed(q, k, v, nn, blob, stream, sws, bs, luts["blocks"], scale, mask=m, valid_len=vl)
            torch.cuda.synchronize()
            assert sfb.stream_status(stream, d, sws) == 0
            check(out.cpu().numpy(), ref, tol)


@pytest.mark.parametrize("d", [32, 96, 128])
@pytest.mark.parametrize("bs", [32, 64])
def test_fused_backward_at_other_head_sizes(d, bs):
    """Head sizes 32, 96 and 128 (tiles cut into slices of 64 features, as in the forward): whole lines and lines cut
    into chunks, with element mask and key padding, against the oracle's backward chain."""
    nb, B, H = 8, 2, 3
    L = nb * bs
    scale = float(1.0 / np.sqrt(d))
    lay = PATTERNS["bigbird"](nb).copy()
    lay[5] = 0
    luts = sfb.build_luts(lay)
    keep = (np.random.default_rng(bs + d).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    mask = sfb.pack_mask(keep)
    valid = np.array([L, L - bs - 7], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=400 + bs + d, bf16=True)
    dO = orc.round_bf16(orc.fill_normal((B, L, H, d), 410))
    q, k, v, do = (dev(x, True) for x in (Q, K, V, dO))
    nn, tn = sfb.to_device(luts["nn_lut"]), sfb.to_device(luts["tn_lut"])
    for masked in (False, True):
        mk, vd = (mask, valid) if masked else (None, None)
        m = None if mk is None else sfb.to_device(mk)
        vl = None if vd is None else sfb.to_device(vd)
        dQ, dK, dV, _ = orc.attention_backward(Q, K, V, dO, luts, bs, scale, mask=mk, valid_len=vd)
        o, lse = forward(q, k, v, luts, bs, scale, mask=m, valid=vl)
        for max_blocks in (None, 3):
            rs = cs = None
            if max_blocks:
                rs, cs = sfb.build_schedule(luts["nn_lut"], nb, max_blocks), sfb.build_schedule(luts["tn_lut"], nb, max_blocks)
                rs["items_dev"], cs["items_dev"] = sfb.to_device(rs["items"]), sfb.to_device(cs["items"])
            dq, dk, dv = sfb.fused_attention_backward(q, k, v, o, do, lse, nn, tn, bs, luts["blocks"], scale, mask=m,
                                                      valid_len=vl, row_sched=rs, col_sched=cs)
            torch.cuda.synchronize()
            for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
                got = got.cpu().numpy()
                assert np.isfinite(got).all()
                assert rel_err(got, want) <= TOL_BF16, (name, masked, max_blocks)
            assert (dq.cpu().numpy()[:, 5 * bs:6 * bs] == 0).all()


@pytest.mark.parametrize("d", [32, 64, 96, 128])
@pytest.mark.parametrize("bs", [32, 64])
def test_fused_backward_fp32_tensors(d, bs):
    """fp32 Q, K, V and dO through the fused backward (true fp32 products): whole lines and lines cut into chunks,
    with element mask and key padding, one table for all heads and one per head, to the fp32 tolerance."""
    nb, B, H = 8, 2, 3
    L = nb * bs
    scale = float(1.0 / np.sqrt(d))
    lay = PATTERNS["bigbird"](nb).copy()
    lay[5] = 0
    lay[:, 6] = 0
    luts = sfb.build_luts(lay)
    keep = (np.random.default_rng(3 * bs + d).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    mask = sfb.pack_mask(keep)
    valid = np.array([L, L - bs - 7], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=500 + bs + d)
    dO = orc.fill_normal((B, L, H, d), 510)
    q, k, v, do = (dev(x, False) for x in (Q, K, V, dO))
    nn, tn = sfb.to_device(luts["nn_lut"]), sfb.to_device(luts["tn_lut"])
    for masked in (False, True):
        mk, vd = (mask, valid) if masked else (None, None)
        m = None if mk is None else sfb.to_device(mk)
        vl = None if vd is None else sfb.to_device(vd)
        dQ, dK, dV, _ = orc.attention_backward(Q, K, V, dO, luts, bs, scale, mask=mk, valid_len=vd)
        o, lse = forward(q, k, v, luts, bs, scale, mask=m, valid=vl)
        for max_blocks in (None, 3):
            rs = cs = None
            if max_blocks:
                rs, cs = sfb.build_schedule(luts["nn_lut"], nb, max_blocks), sfb.build_schedule(luts["tn_lut"], nb, max_blocks)
                rs["items_dev"], cs["items_dev"] = sfb.to_device(rs["items"]), sfb.to_device(cs["items"])
            dq, dk, dv = sfb.fused_attention_backward(q, k, v, o, do, lse, nn, tn, bs, luts["blocks"], scale, mask=m,
                                                      valid_len=vl, row_sched=rs, col_sched=cs)
            torch.cuda.synchronize()
            for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
                got = got.cpu().numpy()
                assert np.isfinite(got).all()
                assert rel_err(got, want) <= TOL_F32, (name, masked, max_blocks)
            assert (dq.cpu().numpy()[:, 5 * bs:6 * bs] == 0).all()
            assert (dk.cpu().numpy()[:, 6 * bs:7 * bs] == 0).all() and (dv.cpu().numpy()[:, 6 * bs:7 * bs] == 0).all()


@pytest.mark.parametrize("d", [32, 96, 128])
@pytest.mark.parametrize("bs", [32, 64])
def test_unfused_bf16_tensors_at_other_head_sizes(d, bs):
    """bf16 Q/K/V/dO with head size 32, 96 or 128 and S, P, dS stored as bf16 (the benched storage): the three
    products, the two-stage fusion and the backward sequence against the oracle run on the bf16-rounded inputs."""
    nb, B, H = 8, 2, 2
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    blocks = luts["blocks"]
    scale = float(1.0 / np.sqrt(d))
    Q, K, V = qkv(B, nb * bs, H, d, seed=5 * d + bs, bf16=True)
    dO = orc.round_bf16(orc.fill_normal((B, nb * bs, H, d), 95 + d))
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, scale)
    q, k, v, do = (dev(x, True) for x in (Q, K, V, dO))
    ld = {name: sfb.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    p = sfb.fusion_attention2(ld["nn_lut"], q, k, bs, blocks, scale, out_dtype=sfb.BF16)
    assert rel_err(p.float().cpu().numpy(), P) <= TOL_BF16
    S = sfb.bst_sgemm_nt(ld["nt_lut"], q, k, bs, blocks, out_dtype=sfb.BF16)
    assert rel_err(S.float().cpu().numpy(), orc.sdd_nt(Q, K, luts["nt_lut"], bs)) <= TOL_BF16
    O = sfb.bst_sgemm_xn(ld["nn_lut"], p, v, nb)
    assert rel_err(O.cpu().numpy(), orc.attention(Q, K, V, luts["nn_lut"], bs, scale)) <= TOL_BF16
    for o in (None, O):
        dq, dk, dv = sfb.attention_backward(q, k, v, do, p, ld, bs, blocks, scale, o=o)
        for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
            # P, dP and dS each pass through memory as bf16: three roundings more than the fused backward carries
            assert rel_err(got.cpu().numpy(), want) <= 2 * TOL_BF16, (name, o is not None)


@pytest.mark.parametrize("d,bf16", [(48, True), (80, True), (8, True), (120, True), (48, False), (80, False), (4, False),
                                    (100, False)])
@pytest.mark.parametrize("bs", [32, 64])
def test_unfused_sequence_and_backward_paths_at_head_sizes_between_the_multiples_of_32(d, bs, bf16):
    """The reference's K64 = false product kernels take any head size that is a multiple of 4
    (openai_blocksparse.h:221-222).  Here: the three products, the two-stage fusion, the backward sequence and the
    fused backward with rows of d elements (multiples of 8 for bf16, of 4 for fp32), run by the kernels of the next
    multiple of 32 with short-row loads and stores; with element mask and key padding in the fused backward."""
    nb, B, H = 8, 2, 3
    L = nb * bs
    tol = TOL_BF16 if bf16 else TOL_F32
    scale = float(1.0 / np.sqrt(d))
    lay = PATTERNS["bigbird"](nb).copy()
    lay[5] = 0
    luts = sfb.build_luts(lay)
    blocks = luts["blocks"]
    Q, K, V = qkv(B, L, H, d, seed=600 + bs + d, bf16=bf16)
    dO = orc.fill_normal((B, L, H, d), 610 + d)
    dO = orc.round_bf16(dO) if bf16 else dO
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, scale)
    q, k, v, do = (dev(x, bf16) for x in (Q, K, V, dO))
    ld = {name: sfb.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    code = sfb.BF16 if bf16 else sfb.F32
    S = sfb.bst_sgemm_nt(ld["nt_lut"], q, k, bs, blocks, out_dtype=code)
    assert rel_err(S.float().cpu().numpy(), orc.sdd_nt(Q, K, luts["nt_lut"], bs)) <= tol
    p = sfb.fusion_attention2(ld["nn_lut"], q, k, bs, blocks, scale, out_dtype=code)
    assert rel_err(p.float().cpu().numpy(), P) <= tol
    O = sfb.bst_sgemm_xn(ld["nn_lut"], p, v, nb)
    assert rel_err(O.cpu().numpy(), orc.attention(Q, K, V, luts["nn_lut"], bs, scale)) <= tol
    assert (O.cpu().numpy()[:, 5 * bs:6 * bs] == 0).all()
    for o in (None, O):
        dq, dk, dv = sfb.attention_backward(q, k, v, do, p, ld, bs, blocks, scale, o=o)
        for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
            # with bf16 storage P, dP and dS each pass through memory as bf16
            assert rel_err(got.cpu().numpy(), want) <= (2 * tol if bf16 else tol), (name, o is None)
    keep = (np.random.default_rng(bs + d).random((blocks, bs, bs)) < 0.8).astype(np.uint8)
    mask, valid = sfb.pack_mask(keep), np.array([L, L - bs - 7], np.int32)
    for mk, vd in ((None, None), (mask, valid)):
        m = None if mk is None else sfb.to_device(mk)
        vl = None if vd is None else sfb.to_device(vd)
        dQ, dK, dV, _ = orc.attention_backward(Q, K, V, dO, luts, bs, scale, mask=mk, valid_len=vd)
        o, lse = forward(q, k, v, luts, bs, scale, mask=m, valid=vl)
        for max_blocks in (None, 3):
            rs = cs = None
            if max_blocks:
                rs, cs = sfb.build_schedule(luts["nn_lut"], nb, max_blocks), sfb.build_schedule(luts["tn_lut"], nb, max_blocks)
                rs["items_dev"], cs["items_dev"] = sfb.to_device(rs["items"]), sfb.to_device(cs["items"])
            dq, dk, dv = sfb.fused_attention_backward(q, k, v, o, do, lse, ld["nn_lut"], ld["tn_lut"], bs, blocks, scale,
                                                      mask=m, valid_len=vl, row_sched=rs, col_sched=cs)
            torch.cuda.synchronize()
            for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
                got = got.cpu().numpy()
                assert np.isfinite(got).all()
                assert rel_err(got, want) <= tol, (name, mk is not None, max_blocks)
            assert (dq.cpu().numpy()[:, 5 * bs:6 * bs] == 0).all()


@pytest.mark.parametrize("bf16,d,heads,streamed,pre_ln", [(True, 40, 4, False, False), (False, 36, 4, False, True),
                                                          (True, 72, 2, True, False), (False, 20, 4, True, False)])
def test_encoder_layer_at_head_sizes_between_the_multiples_of_32(bf16, d, heads, streamed, pre_ln):
    """One encoder layer (both wirings, attention as a scheduled and as a streamed launch) with such head sizes."""
    from test_layer_gpu import T, layer_weights
    B, L, ffn, bs = 2, 512, 256, 64
    n, nb = heads * d, L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    w = layer_weights(n, ffn, 100)
    x = orc.fill_normal((B * L, n), 300)
    oracle = orc.encoder_layer_pre_ln if pre_ln else orc.encoder_layer
    want = oracle(x, w, luts["nn_lut"], B, L, heads, d, ffn, bs, luts["blocks"], operands_bf16=bf16, nthreads=THREADS)
    layer = sfb.EncoderLayer({k: T(v) for k, v in w.items()}, luts, bs, heads, d, ffn,
                             dtype=sfb.BF16 if bf16 else sfb.F32, max_blocks=2, pre_ln=pre_ln, streamed=streamed)
    for _ in range(2):
        got = layer.forward(T(x), B, L).cpu().numpy()
        torch.cuda.synchronize()
        assert rel_err(got, want) <= (TOL_BF16 if bf16 else TOL_F32)
