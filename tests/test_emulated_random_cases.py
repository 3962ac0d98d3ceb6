"""Randomly drawn cases of every attention path on the host model of the kernels (tests/emu_lib.py) against the oracle:
block size, element type, head size (multiples of 32 and sizes between them), number of block rows, batch and heads,
a random block layout (rows and columns without blocks included), with or without an element mask (keeping none, some
or all of the keys) and key padding (valid lengths from 0 to the whole context), the launch form's parameters (chunk
length, stream slots), and the model's lane order and load timing.  A fixed list of seeds, so a failure names its case;
the same generators ran over a thousand seeds while this file was written."""
import numpy as np
import pytest
import torch

import emu_lib
import oracle_lib as orc
from test_emulated_kernels import E, dev, inputs, zeros   # noqa: F401  (E: the module-scoped fixture)


def check(name, got, want, tol, case):
    got = np.asarray(got, np.float64)
    assert np.isfinite(got).all(), (name, case)
    err = np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= tol, (name, err, case, emu_lib.message())


@pytest.mark.parametrize("seed", range(16))
def test_one_table_for_all_heads(E, seed):
    rng = np.random.default_rng(seed)
    bs, bf16 = int(rng.choice([32, 64])), bool(rng.integers(2))
    d = int(rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 96, 104, 128] if bf16 else [4, 12, 32, 36, 64, 68, 96, 100, 128]))
    nb, B, H = int(rng.integers(1, 7)), int(rng.integers(1, 3)), int(rng.integers(1, 4))
    lay = (rng.random((nb, nb)) < rng.choice([0.15, 0.4, 0.8, 1.0])).astype(np.uint32)
    if lay.sum() == 0:
        lay[rng.integers(nb), rng.integers(nb)] = 1
    L = nb * bs
    luts = E.build_luts(lay)
    blocks = luts["blocks"]
    use_mask, use_valid = bool(rng.integers(2)), bool(rng.integers(2))
    mask = E.pack_mask((rng.random((blocks, bs, bs)) < rng.choice([0.0, 0.5, 0.9, 1.0])).astype(np.uint8)) if use_mask else None
    valid = rng.integers(0, L + 1, size=B).astype(np.int32) if use_valid else None
    scale = float(rng.choice([0.05, 0.125, 1.0]))
    Q, K, V, dO = inputs(B, L, H, d, 1000 + seed, bf16, n=4)
    tol = 1e-2 if bf16 else 1e-4
    order, lazy = int(rng.choice([0, 1, int(rng.integers(2, 60))])), bool(rng.integers(2))
    emu_lib.configure(order=order, lazy_loads=lazy)
    case = dict(seed=seed, bs=bs, d=d, bf16=bf16, nb=nb, B=B, H=H, mask=use_mask, valid=use_valid, scale=scale, order=order,
                lazy=lazy)
    q, k, v, do = (dev(x, bf16) for x in (Q, K, V, dO))
    nn, tn, nt = (E.to_device(luts[name]) for name in ("nn_lut", "tn_lut", "nt_lut"))
    md, vd = (None if mask is None else E.to_device(mask)), (None if valid is None else E.to_device(valid))
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, mask=mask, valid_len=valid)
    check("plain", E.fused_attention(q, k, v, nn, bs, blocks, scale, mask=md, valid_len=vd).float().numpy(), want, tol, case)
    max_blocks = int(rng.integers(1, 5))
    sched = E.build_schedule(luts["nn_lut"], nb, max_blocks)
    ws = zeros(E.schedule_workspace_bytes(sched, B, H, bs, d))
    for _ in range(2):
        o, lse = E.fused_attention_forward_lse(q, k, v, nn, E.to_device(sched["items"]), sched, ws, bs, blocks, scale, mask=md,
                                               valid_len=vd)
        check("scheduled", o.numpy(), want, tol, case)
    stream = E.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=int(rng.choice([1, 3, 8, 40])), d=d, bf16=bf16,
                            masked=use_mask or use_valid, level=bool(rng.integers(2)))
    sw = zeros(E.stream_workspace_bytes(stream, d))
    for _ in range(2):
        got = E.fused_attention_streamed(q, k, v, nn, E.to_device(stream["blob"]), stream, sw, bs, blocks, scale, mask=md,
                                         valid_len=vd)
        assert E.stream_status(stream, d, sw) == 0, case
        check("streamed", got.float().numpy(), want, tol, case)
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, scale, mask=mask, valid_len=valid)
    rs = cs = None
    if rng.integers(2):
        rs, cs = E.build_schedule(luts["nn_lut"], nb, max_blocks), E.build_schedule(luts["tn_lut"], nb, max_blocks)
        rs["items_dev"], cs["items_dev"] = E.to_device(rs["items"]), E.to_device(cs["items"])
    dq, dk, dv = E.fused_attention_backward(q, k, v, o, do, lse, nn, tn, bs, blocks, scale, mask=md, valid_len=vd, row_sched=rs,
                                            col_sched=cs)
    for name, g, w in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        if np.abs(w).max() > 0:
            check("fused backward " + name, g.numpy(), w, 2 * tol if bf16 else tol, case)
        else:
            assert (g.numpy() == 0).all(), (name, case)
    code = E.BF16 if bf16 else E.F32
    p2 = E.fusion_attention2(nn, q, k, bs, blocks, scale, mask=md, valid_len=vd, out_dtype=code)
    check("two-stage fusion", p2.float().numpy(), P, tol, case)
    S = E.bst_sgemm_nt(nt, q, k, bs, blocks, out_dtype=code)
    check("sdd", S.float().numpy(), orc.sdd_nt(Q, K, luts["nt_lut"], bs), tol, case)
    O = E.bst_sgemm_xn(nn, p2, v, nb)
    check("dsd", O.numpy(), want, 2 * tol if bf16 else tol, case)
    ld = {"nt_lut": nt, "nn_lut": nn, "tn_lut": tn}
    dq, dk, dv = E.attention_backward(q, k, v, do, p2, ld, bs, blocks, scale, o=O if rng.integers(2) else None)
    for name, g, w in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        if np.abs(w).max() > 0:
            check("unfused backward " + name, g.numpy(), w, 3 * tol if bf16 else tol, case)


@pytest.mark.parametrize("seed", range(6))
def test_one_table_and_mask_per_head(E, seed):
    rng = np.random.default_rng(seed)
    bs, bf16 = int(rng.choice([32, 64])), bool(rng.integers(2))
    d = int(rng.choice([32, 64, 96, 128] + ([40, 72] if bf16 else [36, 100])))
    nb, B, H = int(rng.integers(2, 11)), int(rng.integers(1, 3)), int(rng.integers(2, 4))
    base = (rng.random((nb, nb)) < rng.choice([0.1, 0.3, 0.6])).astype(np.uint32)
    if base.sum() == 0:
        base[0, 0] = 1
    per_head = [E.build_luts(base[:, rng.permutation(nb)][rng.permutation(nb)]) for _ in range(H)]   # equal block counts
    blocks = per_head[0]["blocks"]
    L = nb * bs
    nn, nt, tn = (np.concatenate([p[name] for p in per_head]) for name in ("nn_lut", "nt_lut", "tn_lut"))
    use_mask, use_valid = bool(rng.integers(2)), bool(rng.integers(2))
    words = [E.pack_mask((rng.random((blocks, bs, bs)) < 0.8).astype(np.uint8)) for _ in range(H)] if use_mask else None
    mask = np.concatenate(words) if use_mask else None
    valid = rng.integers(1, L + 1, size=B).astype(np.int32) if use_valid else None
    mask_heads = H if use_mask else 1
    scale = float(rng.choice([0.125, 0.3]))
    Q, K, V, dO = inputs(B, L, H, d, 2000 + seed, bf16, n=4)
    tol = 1e-2 if bf16 else 1e-4
    order, lazy = int(rng.choice([0, 1, int(rng.integers(2, 60))])), bool(rng.integers(2))
    emu_lib.configure(order=order, lazy_loads=lazy)
    case = dict(seed=seed, bs=bs, d=d, bf16=bf16, nb=nb, B=B, H=H, blocks=blocks, mask=use_mask, valid=use_valid, order=order,
                lazy=lazy)
    q, k, v, do = (dev(x, bf16) for x in (Q, K, V, dO))
    nnd, tnd, ntd = E.to_device(nn), E.to_device(tn), E.to_device(nt)
    md, vd = (None if mask is None else E.to_device(mask)), (None if valid is None else E.to_device(valid))
    want = orc.attention(Q, K, V, nn, bs, scale, mask=mask, valid_len=valid, lut_heads=H, mask_heads=mask_heads, blocks=blocks)
    got = E.fused_attention(q, k, v, nnd, bs, blocks, scale, mask=md, valid_len=vd, lut_heads=H, mask_heads=mask_heads)
    check("plain", got.float().numpy(), want, tol, case)
    sched = E.build_schedule_heads(nn, nb, H, int(rng.integers(1, 6)))
    ws = zeros(E.schedule_workspace_bytes(sched, B, H, bs, d))
    for _ in range(2):
        got = E.fused_attention_scheduled_heads(q, k, v, nnd, E.to_device(sched["items"]), sched, ws, bs, blocks, scale, mask=md,
                                                valid_len=vd, mask_heads=mask_heads)
        check("scheduled, work items per head", got.float().numpy(), want, tol, case)
    stream = E.build_stream(nn, nb, B, H, bs, lut_heads=H, wg_slots=int(rng.choice([2, 8, 40])), d=d, bf16=bf16,
                            masked=use_mask or use_valid, level=bool(rng.integers(2)))
    sw = zeros(E.stream_workspace_bytes(stream, d))
    lse = emu_lib.empty((B, H, L), torch.float32, fill=7.0)
    for _ in range(2):
        o = E.fused_attention_streamed(q, k, v, nnd, E.to_device(stream["blob"]), stream, sw, bs, blocks, scale, mask=md,
                                       valid_len=vd, mask_heads=mask_heads, lse=lse)
        assert E.stream_status(stream, d, sw) == 0, case
        check("streamed", o.numpy(), want, tol, case)
    dq, dk, dv = E.fused_attention_backward(q, k, v, o, do, lse, nnd, tnd, bs, blocks, scale, mask=md, valid_len=vd,
                                            mask_heads=mask_heads, lut_heads=H)
    for h in range(H):
        one = lambda x: np.ascontiguousarray(x[:, :, h:h + 1])   # noqa: E731
        dQ, dK, dV, _ = orc.attention_backward(one(Q), one(K), one(V), one(dO), per_head[h], bs, scale,
                                               mask=None if words is None else words[h], valid_len=valid)
        for name, g, w in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
            if np.abs(w).max() > 0:
                check("fused backward %s, head %d" % (name, h), g.numpy()[:, :, h:h + 1], w, 2 * tol if bf16 else tol, case)
    code = E.BF16 if bf16 else E.F32
    S = E.bst_sgemm_nt(ntd, q, k, bs, blocks, out_dtype=code, lut_heads=H)
    S_want = orc.sdd_nt(Q, K, nt, bs, lut_heads=H)
    check("sdd", S.float().numpy(), S_want, tol, case)
    row_major = None if words is None else E.to_device(np.concatenate([E.transpose_mask(w, blocks, bs) for w in words]))
    P = E.BlocksparseMaskedSoftmax(nnd, row_major, S, nb, scale, out_dtype=code, valid_len=vd, lut_heads=H, mask_heads=mask_heads)
    P_want = orc.masked_softmax(S_want, nn, nb, scale, mask=mask, valid_len=valid, lut_heads=H, mask_heads=mask_heads)
    check("softmax", P.float().numpy(), P_want, 2 * tol if bf16 else tol, case)
    p2 = E.fusion_attention2(nnd, q, k, bs, blocks, scale, mask=md, valid_len=vd, out_dtype=code, lut_heads=H, mask_heads=mask_heads)
    check("two-stage fusion", p2.float().numpy(), P_want, tol, case)
    check("dsd", E.bst_sgemm_xn(nnd, p2, v, nb, lut_heads=H).numpy(), want, 2 * tol if bf16 else tol, case)
    if p2.dtype == v.dtype:   # the same product over work items, lines cut at a random length
        cut = int(rng.integers(1, 5))
        sched = E.build_schedule_heads(nn, nb, H, cut) if H > 1 else E.build_schedule(nn, nb, cut)
        ws = emu_lib.empty((max(E.dsd_workspace_bytes(sched, B, H, bs, d), 256),), torch.uint8, fill=0xFF)
        got = E.bst_sgemm_xn_scheduled(nnd, p2, v, nb, E.to_device(sched["items"]), sched, ws, lut_heads=H)
        check("dsd over work items", got.numpy(), want, 2 * tol if bf16 else tol, dict(case, cut=cut))


@pytest.mark.parametrize("seed", range(8))
def test_encoder_layer(E, seed):
    """One encoder layer with random widths (hidden = heads x head size, FFN width down to 4), wiring (post- / pre-LN),
    attention launch (scheduled with a random chunk length, streamed), Q/K/V as one product or three, over a random
    layout that may leave block-rows empty."""
    rng = np.random.default_rng(seed)
    bf16, bs = bool(rng.integers(2)), int(rng.choice([32, 64]))
    d = int(rng.choice([32, 64, 96] + ([40, 8] if bf16 else [36, 20])))
    H, B, nb = int(rng.integers(1, 5)), int(rng.integers(1, 3)), int(rng.integers(1, 6))
    ffn = int(rng.choice([4, 64, 100, 256, 516]))
    L, n = nb * bs, H * d
    lay = (rng.random((nb, nb)) < rng.choice([0.3, 0.7, 1.0])).astype(np.uint32)
    if lay.sum() == 0:
        lay[0, 0] = 1
    luts = E.build_luts(lay)
    pre_ln, streamed, merge = bool(rng.integers(2)), bool(rng.integers(2)), bool(rng.integers(2))
    max_blocks = int(rng.choice([0, 1, 3, 16]))
    emu_lib.configure(order=int(rng.choice([0, 1, int(rng.integers(2, 60))])), lazy_loads=bool(rng.integers(2)))
    case = dict(seed=seed, bf16=bf16, bs=bs, d=d, H=H, B=B, nb=nb, ffn=ffn, pre_ln=pre_ln, streamed=streamed, merge=merge,
                max_blocks=max_blocks)
    shapes = [("wq", (n, n)), ("wk", (n, n)), ("wv", (n, n)), ("wo", (n, n)), ("w1", (n, ffn)), ("w2", (ffn, n)),
              ("bq", (n,)), ("bk", (n,)), ("bv", (n,)), ("bo", (n,)), ("b1", (ffn,)), ("b2", (n,)),
              ("ln1_g", (n,)), ("ln1_b", (n,)), ("ln2_g", (n,)), ("ln2_b", (n,))]
    w = {name: orc.fill_normal(shape, 100 + 20 * seed + i, 0.1 if name[0] == "b" else 0.02) for i, (name, shape) in enumerate(shapes)}
    w["ln1_g"], w["ln2_g"] = w["ln1_g"] + 1, w["ln2_g"] + 1
    x = orc.fill_normal((B * L, n), 300 + seed)
    oracle = orc.encoder_layer_pre_ln if pre_ln else orc.encoder_layer
    want = oracle(x, w, luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"], operands_bf16=bf16, nthreads=4)
    kw = dict(dtype=E.BF16 if bf16 else E.F32, pre_ln=pre_ln, max_blocks=max_blocks)
    if streamed:
        kw["streamed"] = True
    else:
        kw["merge_qkv"] = merge
    layer = E.EncoderLayer({name: dev(a) for name, a in w.items()}, luts, bs, H, d, ffn, **kw)
    for _ in range(2):
        check("encoder layer", layer.forward(dev(x), B, L).numpy(), want, 1e-2 if bf16 else 1e-4, case)
