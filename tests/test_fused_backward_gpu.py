"""Fused backward of the attention (two kernels, nothing sparse in memory) and the forward's log-sum-exp output
against the CPU oracle's backward chain, through the C ABI."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, dev, qkv, rel_err
from sfb import sfb

pytestmark = pytest.mark.gpu


def forward(q, k, v, luts, bs, scale, mask=None, valid=None, max_blocks=4):
    B, L, H, d = q.shape
    sched = sfb.build_schedule(luts["nn_lut"], L // bs, max_blocks)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    return sfb.fused_attention_forward_lse(q, k, v, sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"]), sched,
                                           ws, bs, luts["blocks"], scale, mask=mask, valid_len=valid)


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("pattern,masked", [("causal", True), ("bigbird", False), ("bigbird", True), ("strided", False)])
def test_fused_backward_matches_oracle(pattern, masked, bs):
    nb, B, H, d = 16, 2, 3, 64
    lay = PATTERNS[pattern](nb).copy()
    if pattern == "bigbird":
        lay[5] = 0      # a block-row without blocks
        lay[:, 9] = 0   # a block-column without blocks
    luts = sfb.build_luts(lay)
    mask = valid = None
    if masked:
        if pattern == "causal":
            mask = sfb.pack_mask(sfb.element_mask(luts["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG))
        else:
            keep = (np.random.default_rng(bs).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
            mask = sfb.pack_mask(keep)
        valid = np.array([nb * bs, nb * bs - bs - 7], np.int32)
    Q, K, V = qkv(B, nb * bs, H, d, seed=200 + bs, bf16=True)
    dO = orc.round_bf16(orc.fill_normal((B, nb * bs, H, d), 210))
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, 0.125, mask=mask, valid_len=valid)
    q, k, v, do = (dev(x, True) for x in (Q, K, V, dO))
    m = None if mask is None else sfb.to_device(mask)
    vl = None if valid is None else sfb.to_device(valid)
    o, lse = forward(q, k, v, luts, bs, 0.125, mask=m, valid=vl)
    want_o = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, mask=mask, valid_len=valid)
    assert rel_err(o.cpu().numpy(), want_o) <= TOL_BF16

    # the log-sum-exp rebuilds the oracle's probabilities: P = exp2(S scale log2e - lse)
    S = orc.sdd_nt(Q, K, luts["nt_lut"], bs)
    lse_np = lse.cpu().numpy()
    worst = 0.0
    for blk, (r, _) in enumerate(luts["nt_lut"]):
        rebuilt = np.exp2(S[:, :, blk] * (0.125 * np.log2(np.e)) - lse_np[:, :, r * bs:(r + 1) * bs, None])
        kept = P[:, :, blk] > 0
        worst = max(worst, float(np.abs(np.where(kept, rebuilt - P[:, :, blk], 0)).max()))
    # the bf16 kernel sums the probabilities as it uses them, rounded to bf16: its denominator carries that noise
    assert worst <= 2e-3 * P.max()

    nn, tn = sfb.to_device(luts["nn_lut"]), sfb.to_device(luts["tn_lut"])
    results = []
    for max_blocks in (None, 3, 100):   # whole lines in index order; lines cut into chunks of 3 blocks; sorted only
        rs = cs = None
        if max_blocks:
            rs, cs = sfb.build_schedule(luts["nn_lut"], nb, max_blocks), sfb.build_schedule(luts["tn_lut"], nb, max_blocks)
            rs["items_dev"], cs["items_dev"] = sfb.to_device(rs["items"]), sfb.to_device(cs["items"])
            assert (max_blocks == 3) == (rs["n_parts"] > 0 and cs["n_parts"] > 0)
        dq, dk, dv = sfb.fused_attention_backward(q, k, v, o, do, lse, nn, tn, bs, luts["blocks"], 0.125, mask=m,
                                                  valid_len=vl, row_sched=rs, col_sched=cs)
        torch.cuda.synchronize()
        for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
            got = got.cpu().numpy()
            assert np.isfinite(got).all()
            assert rel_err(got, want) <= TOL_BF16, (name, max_blocks)
        if pattern == "bigbird":
            assert (dq.cpu().numpy()[:, 5 * bs:6 * bs] == 0).all()
            assert (dk.cpu().numpy()[:, 9 * bs:10 * bs] == 0).all() and (dv.cpu().numpy()[:, 9 * bs:10 * bs] == 0).all()
        results.append((dq, dk, dv))
    # the order in which whole lines are handed out does not change a bit; and a second call with split lines
    # gives the same bits as the first (the partial records are added in chunk order)
    for x, y in zip(results[0], results[2]):
        assert torch.equal(x, y)
    rs, cs = sfb.build_schedule(luts["nn_lut"], nb, 3), sfb.build_schedule(luts["tn_lut"], nb, 3)
    rs["items_dev"], cs["items_dev"] = sfb.to_device(rs["items"]), sfb.to_device(cs["items"])
    again = sfb.fused_attention_backward(q, k, v, o, do, lse, nn, tn, bs, luts["blocks"], 0.125, mask=m, valid_len=vl,
                                         row_sched=rs, col_sched=cs)
    for x, y in zip(results[1], again):
        assert torch.equal(x, y)


@pytest.mark.parametrize("bs", [32, 64])
def test_fused_backward_per_head_tables_and_masks(bs):
    """One look-up table and one element mask per head (the reference's `fixed` pattern): forward with its
    log-sum-exp through the streamed entry point, backward with every line done whole; the oracle head by head."""
    nb, B, H, d = 8, 2, 4, 64
    L = nb * bs
    lays = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lays[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    assert all(l["blocks"] == blocks for l in per_head)
    assert any((per_head[0]["nn_lut"] != per_head[h]["nn_lut"]).any() for h in range(1, H))
    nn = np.concatenate([l["nn_lut"] for l in per_head])
    tn = np.concatenate([l["tn_lut"] for l in per_head])
    rng = np.random.default_rng(bs)
    masks = []
    for h in range(H):
        keep = (rng.random((blocks, bs, bs)) < 0.8).astype(np.uint8)
        keep[:, np.arange(bs), np.arange(bs)] = 1
        masks.append(sfb.pack_mask(keep))
    mask = np.concatenate(masks)
    valid = np.array([L, L - bs - 7], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=300 + bs, bf16=True)
    dO = orc.round_bf16(orc.fill_normal((B, L, H, d), 310))
    q, k, v, do = (dev(x, True) for x in (Q, K, V, dO))
    m, vl = sfb.to_device(mask), sfb.to_device(valid)
    stream = sfb.build_stream(nn, nb, B, H, bs, lut_heads=H)
    ws = torch.zeros(sfb.stream_workspace_bytes(stream, d), dtype=torch.uint8, device="cuda")
    o = torch.empty((B, L, H, d), device="cuda")
    lse = torch.empty((B, H, L), device="cuda")
    sfb.fused_attention_streamed(q, k, v, sfb.to_device(nn), sfb.to_device(stream["blob"]), stream, ws, bs, blocks,
                                 0.125, mask=m, valid_len=vl, mask_heads=H, out=o, lse=lse)
    dq, dk, dv = sfb.fused_attention_backward(q, k, v, o, do, lse, sfb.to_device(nn), sfb.to_device(tn), bs, blocks,
                                              0.125, mask=m, valid_len=vl, mask_heads=H, lut_heads=H)
    torch.cuda.synchronize()
    assert sfb.stream_status(stream, d, ws) == 0
    for h in range(H):
        one = lambda x: np.ascontiguousarray(x[:, :, h:h + 1])
        dQ, dK, dV, _ = orc.attention_backward(one(Q), one(K), one(V), one(dO), per_head[h], bs, 0.125, mask=masks[h],
                                               valid_len=valid)
        for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
            assert rel_err(got[:, :, h:h + 1].cpu().numpy(), want) <= TOL_BF16, (name, h)
    # work items describe one layout only
    rs = sfb.build_schedule(per_head[0]["nn_lut"], nb, 3)
    rs["items_dev"] = sfb.to_device(rs["items"])
    with pytest.raises(sfb.SfbError) as e:
        sfb.fused_attention_backward(q, k, v, o, do, lse, sfb.to_device(nn), sfb.to_device(tn), bs, blocks, 0.125,
                                     row_sched=rs, lut_heads=H)
    assert e.value.status == 4


def test_fused_backward_rejects_other_dtypes():
    q = torch.zeros((1, 64, 1, 64), device="cuda", dtype=torch.float16)
    lut = sfb.to_device(np.zeros((2, 2), np.uint32))
    with pytest.raises(sfb.SfbError) as e:
        sfb.fused_attention_backward(q, q, q, q, q, torch.zeros((1, 1, 64), device="cuda"), lut, lut, 64, 1, 0.125)
    assert e.value.status == 5


def test_fused_backward_full_size_identities():
    """C4 workload (BigBird B4 H12 L4096, 622 blocks), scheduled with split global rows and columns: O is linear in V
    and S is bilinear in Q, K, hence <dV, V> = <dO, O> and <dQ, Q> = <dK, K>; every gradient row is written."""
    import bench
    pattern, B, H, L, d, bs, _ = bench.WORKLOADS["c4"]
    nb = L // bs
    luts = sfb.build_luts(bench.make_layout(sfb, pattern, nb))
    torch.manual_seed(5)
    q, k, v, do = (torch.randn((B, L, H, d), device="cuda").to(torch.bfloat16) for _ in range(4))
    o, lse = forward(q, k, v, luts, bs, 0.125, max_blocks=16)
    rs, cs = sfb.build_schedule(luts["nn_lut"], nb, 16), sfb.build_schedule(luts["tn_lut"], nb, 16)
    assert rs["n_parts"] > 0 and cs["n_parts"] > 0
    rs["items_dev"], cs["items_dev"] = sfb.to_device(rs["items"]), sfb.to_device(cs["items"])
    dq, dk, dv = sfb.fused_attention_backward(q, k, v, o, do, lse, sfb.to_device(luts["nn_lut"]),
                                              sfb.to_device(luts["tn_lut"]), bs, luts["blocks"], 0.125, row_sched=rs,
                                              col_sched=cs)
    torch.cuda.synchronize()
    dot = lambda a, b: float((a.double() * b.double()).sum())
    dv_v, do_o = dot(dv, v), dot(do, o)
    dq_q, dk_k = dot(dq, q), dot(dk, k)
    scale_v = float((dv.double() * v.double()).abs().sum())
    scale_q = float((dq.double() * q.double()).abs().sum())
    # P is rounded to bf16 inside both kernels and O inside the forward: the identities hold to that rounding
    assert abs(dv_v - do_o) <= 2e-3 * scale_v
    assert abs(dq_q - dk_k) <= 2e-3 * scale_q
    for g in (dq, dk, dv):
        assert torch.isfinite(g).all() and float(g.abs().amax(dim=(0, 2, 3)).min()) > 0
