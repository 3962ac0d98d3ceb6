"""Cases of the block-sparse x dense products launched over work items (sfb_dsd_xn_scheduled) against the CPU oracle
and against the launch by lines.  `S` is the binding (capi of the device library or of its host build), `dev` puts a
numpy array where that library reads it, `poisoned` gives device bytes that are not zero (the workspace needs no
initial contents)."""
import numpy as np

import oracle_lib as orc

TOL_F32 = 1e-4
ERR_SHAPE, ERR_DTYPE, ERR_WORKSPACE = 4, 5, 9   # SFB_ERR_* of the C header


def rel_err(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def layouts(S, nb, heads):
    """One BigBird layout (global first and last block: lines of nb blocks beside lines of a few), or one layout per
    head of the reference's `fixed` pattern with equal block counts."""
    if heads == 1:
        lay = S.layout_bigbird(nb, 1, 1, True, S.bigbird_draw(nb, 1, 1, True, 1, 5)).copy()
        lay[2, :] = 0
        lay[2, 2] = 1          # a short row
        lay[:, 5] = 0          # a key-block column without blocks
        lay[5, :] = 0          # and a block-row without blocks
        return [lay]
    lays = S.layout_fixed(heads, nb, 4, causal=True)
    return [lays[h] for h in range(heads)]


def products(S, dev, poisoned, bs, d, bf16, heads_with_own_table=1, max_blocks=3, nb=8, B=2, H=3):
    """NN and TN products over work items cut at max_blocks key blocks: equal to the oracle's, zero where a line has no
    blocks, and no element of the result left unwritten."""
    import torch
    per_head = heads_with_own_table > 1
    if per_head:
        H = heads_with_own_table
    luts = [S.build_luts(lay) for lay in layouts(S, nb, heads_with_own_table)]
    blocks = luts[0]["blocks"]
    assert all(l["blocks"] == blocks for l in luts)
    rounded = orc.round_bf16 if bf16 else (lambda x: x)
    A = rounded(orc.fill_normal((B, H, blocks, bs, bs), 21))
    X = rounded(orc.fill_normal((B, nb * bs, H, d), 22))

    def sparse(x):
        t = dev(np.ascontiguousarray(x))
        return t.to(torch.bfloat16) if bf16 else t

    a, x = sparse(A), sparse(X)
    for op, key, oracle in ((S.NN_OP, "nn_lut", orc.dsd_nn), (S.TN_OP, "tn_lut", orc.dsd_tn)):
        lut = np.concatenate([l[key] for l in luts])
        want = oracle(A, X, lut, lut_heads=len(luts))
        if per_head:
            sched = S.build_schedule_heads(lut, nb, H, max_blocks)
        else:
            sched = S.build_schedule(lut, nb, max_blocks)
        assert sched["n_parts"] > 0, "some line is cut"
        ws = poisoned(S.dsd_workspace_bytes(sched, B, H, bs, d))
        out = dev(np.full((B, nb * bs, H, d), 7.0, np.float32))
        S.bst_sgemm_xn_scheduled(S.to_device(lut), a, x, nb, S.to_device(sched["items"]), sched, ws, op=op,
                                 lut_heads=len(luts), c=out)
        got = out.cpu().numpy()
        assert rel_err(got, want) <= TOL_F32, (op, rel_err(got, want))   # exact inputs, fp32 sums on both sides
        if not per_head:
            assert (got[:, 5 * bs:6 * bs] == 0).all()
        plain = S.bst_sgemm_xn(S.to_device(lut), a, x, nb, op=op, lut_heads=len(luts)).cpu().numpy()
        assert rel_err(got, plain) <= TOL_F32
        # uncut: every item is a whole line, no workspace
        whole = S.build_schedule_heads(lut, nb, H, nb) if per_head else S.build_schedule(lut, nb, nb)
        assert whole["n_parts"] == 0
        got = S.bst_sgemm_xn_scheduled(S.to_device(lut), a, x, nb, S.to_device(whole["items"]), whole, None, op=op,
                                       lut_heads=len(luts)).cpu().numpy()
        assert (got == plain).all(), "the same sums in the same order"


def argument_errors(S, dev, poisoned):
    import torch
    bs, d, nb, B, H = 64, 64, 8, 1, 2
    luts = S.build_luts(layouts(S, nb, 1)[0])
    blocks = luts["blocks"]
    a = dev(np.zeros((B, H, blocks, bs, bs), np.float32))
    x = dev(np.zeros((B, nb * bs, H, d), np.float32))
    sched = S.build_schedule(luts["nn_lut"], nb, 3)
    items, lut = S.to_device(sched["items"]), S.to_device(luts["nn_lut"])
    need = S.dsd_workspace_bytes(sched, B, H, bs, d)
    assert need == B * H * sched["n_parts"] * bs * d * 4

    def status(call):
        try:
            call()
        except S.SfbError as e:
            return e.status
        return 0

    ws = poisoned(need)
    assert status(lambda: S.bst_sgemm_xn_scheduled(lut, a, x, nb, items, sched, ws)) == 0
    assert status(lambda: S.bst_sgemm_xn_scheduled(lut, a, x, nb, items, sched, None)) == ERR_WORKSPACE
    assert status(lambda: S.bst_sgemm_xn_scheduled(lut, a, x, nb, items, sched, ws[:need - 256])) == ERR_WORKSPACE
    assert status(lambda: S.bst_sgemm_xn_scheduled(lut, a, x, nb, items, sched, ws[16:])) == ERR_WORKSPACE
    assert status(lambda: S.bst_sgemm_xn_scheduled(lut, a.to(torch.bfloat16), x, nb, items, sched, ws)) == ERR_DTYPE
    bad = dict(sched, n_heavy=sched["n_items"])
    assert status(lambda: S.bst_sgemm_xn_scheduled(lut, a, x, nb, items, bad, ws)) == ERR_SHAPE
