"""Planned launches (resident work-groups walking host-built lists of work items, sfb_build_plan +
sfb_fused_attention_planned) against the CPU oracle and against the scheduled entry point."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, qkv, rel_err
from sfb import sfb

pytestmark = pytest.mark.gpu
THREADS = 16


def run_planned(Q, K, V, nn_lut, nb, bs, blocks, scale, bf16, max_blocks=None, lut_heads=1, mask=None, valid_len=None,
                mask_heads=1, wg_slots=None, out_bf16=False, want_lse=False, launches=2):
    B, L, H, d = Q.shape
    plan = sfb.build_plan(nn_lut, nb, B, H, max_blocks=max_blocks, lut_heads=lut_heads, wg_slots=wg_slots)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(plan, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    nn, plan_dev = sfb.to_device(nn_lut), sfb.to_device(plan["plan"])
    m = None if mask is None else sfb.to_device(mask)
    vl = None if valid_len is None else sfb.to_device(np.asarray(valid_len, np.int32))
    outs = []
    for _ in range(launches):   # later launches find the arrival counters as the first one left them
        out = torch.full((B, L, H, d), 7.0, device="cuda", dtype=torch.bfloat16 if out_bf16 else torch.float32)
        lse = torch.full((B, H, L), 7.0, device="cuda") if want_lse else None
        sfb.fused_attention_planned(q, k, v, nn, plan_dev, plan, ws, bs, blocks, scale, mask=m, valid_len=vl,
                                    mask_heads=mask_heads, out=out, lse=lse)
        torch.cuda.synchronize()
        outs.append(out)
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    assert int(ws[:max(4 * B * H * plan["n_slots"], 4)].view(torch.int32).abs().sum()) == 0
    return (outs[0], lse, plan) if want_lse else (outs[0], plan)


@pytest.mark.parametrize("bf16", [True, False])
def test_c4_bigbird_planned(bf16):
    B, H, L, d, bs = 4, 12, 4096, 64, 64
    luts = sfb.build_luts(PATTERNS["bigbird"](L // bs))
    Q, K, V = qkv(B, L, H, d, seed=404, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    got, plan = run_planned(Q, K, V, luts["nn_lut"], L // bs, bs, luts["blocks"], 0.125, bf16)
    got = got.cpu().numpy()
    assert plan["n_parts"] > 0
    diff = np.abs(got.astype(np.float64) - want).max(axis=(1, 3)) / np.abs(want).max(axis=(1, 3))
    print("max_blocks", plan["max_blocks"], "stride", plan["plan_stride"], "worst (batch, head) error %.3e" % diff.max(),
          flush=True)
    assert np.isfinite(got).all() and diff.max() <= (TOL_BF16 if bf16 else TOL_F32)


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("max_blocks,wg_slots", [(3, 16), (8, 1024), (1, 7), (1000, 64)])
def test_planned_masks_padding_split_rows(bf16, max_blocks, wg_slots):
    bs, nb, B, H, d = 64, 16, 2, 3, 64
    L = bs * nb
    lay = PATTERNS["bigbird"](nb).copy()
    lay[5] = 0   # an empty block-row
    luts = sfb.build_luts(lay)
    keep = (np.random.default_rng(7).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    mask = sfb.pack_mask(keep)
    valid = np.array([L, L - 100], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=95, bf16=bf16)
    tol = TOL_BF16 if bf16 else TOL_F32
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, mask=mask, valid_len=valid, nthreads=THREADS)
    got, _ = run_planned(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, bf16, max_blocks=max_blocks,
                         mask=mask, valid_len=valid, wg_slots=wg_slots)
    assert rel_err(got.cpu().numpy(), want) <= tol
    assert (got[:, 5 * bs:6 * bs] == 0).all()
    # the same layout without mask and padding takes the kernels' other instantiation
    plain = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    got, _ = run_planned(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, bf16, max_blocks=max_blocks,
                         wg_slots=wg_slots)
    assert rel_err(got.cpu().numpy(), plain) <= tol


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("bs", [32, 64])
def test_planned_per_head_luts_and_masks(bf16, bs):
    """The reference's `fixed` pattern gives every head its own layout (fixed_fusion_test.cu:38-39, 58-106)."""
    nb, B, H, d = 16, 3, 4, 64
    L = bs * nb
    lay = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lay[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    assert all(p["blocks"] == blocks for p in per_head)
    assert any(not np.array_equal(per_head[0]["nn_lut"], p["nn_lut"]) for p in per_head[1:])
    nn = np.concatenate([p["nn_lut"] for p in per_head])
    masks = np.concatenate([sfb.pack_mask(sfb.element_mask(p["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG)) for p in per_head])
    Q, K, V = qkv(B, L, H, d, seed=80, bf16=bf16)
    want = orc.attention(Q, K, V, nn, bs, 0.125, mask=masks, lut_heads=H, mask_heads=H, blocks=blocks, nthreads=THREADS)
    for max_blocks in (2, 100):
        got, plan = run_planned(Q, K, V, nn, nb, bs, blocks, 0.125, bf16, max_blocks=max_blocks, lut_heads=H,
                                mask=masks, mask_heads=H, wg_slots=40)
        live = plan["plan"]["count"] != sfb.PLAN_END
        assert live.sum() == B * sum(len(sfb.build_schedule(p["nn_lut"], nb, max_blocks)["items"]) for p in per_head)
        assert rel_err(got.cpu().numpy(), want) <= (TOL_BF16 if bf16 else TOL_F32)


def test_planned_bf16_output_and_lse_match_the_scheduled_entry():
    bs, nb, B, H, d = 64, 32, 2, 4, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    Q, K, V = qkv(B, L, H, d, seed=77, bf16=True)
    got, lse, plan = run_planned(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, True, max_blocks=8,
                                 out_bf16=True, want_lse=True)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    sched = sfb.build_schedule(luts["nn_lut"], nb, 8)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    o32, lse2 = sfb.fused_attention_forward_lse(q, k, v, sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"]),
                                                sched, ws, bs, luts["blocks"], 0.125)
    torch.cuda.synchronize()
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    assert rel_err(got.float().cpu().numpy(), want) <= TOL_BF16
    # same kernels and the same cuts: only the order in which chunks of a split row arrive may differ
    assert rel_err(got.float().cpu().numpy(), o32.cpu().numpy()) <= 2.0 ** -7
    assert torch.allclose(lse, lse2, rtol=0, atol=1e-3)


def test_planned_overflowing_scores_take_the_general_loop():
    """Scores that grow along the row by more than 2^100 in probability: the loop without running maximum
    overflows, notices, and the item is redone with the running maximum."""
    bs, nb, B, H, d = 64, 8, 1, 2, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["full"](nb))
    Q, K, V = qkv(B, L, H, d, seed=91, bf16=True)
    K = orc.round_bf16(K * (1.0 + 3.0 * np.arange(L, dtype=np.float32)[None, :, None, None] / L))
    Q = orc.round_bf16(Q * 24.0)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    s = np.einsum("lhd,mhd->hlm", Q[0].astype(np.float64), K[0].astype(np.float64)) * 0.125 * np.log2(np.e)
    assert (s.max(axis=2) - s[:, :, :bs].max(axis=2)).max() > 110   # later blocks exceed the first one's maximum by 2^110
    got, _ = run_planned(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, True, wg_slots=8)
    got = got.cpu().numpy()
    assert np.isfinite(got).all()
    assert rel_err(got, want) <= TOL_BF16

    # the unscheduled and the scheduled entry points run the same loops
    from gpu_common import run_fused
    assert rel_err(run_fused(Q, K, V, luts, bs, 0.125, bf16=True), want) <= TOL_BF16
    assert rel_err(run_fused(Q, K, V, luts, bs, 0.125, bf16=True, max_blocks=3), want) <= TOL_BF16
