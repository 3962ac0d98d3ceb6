"""Streamed launches (resident work-groups walking host-built streams of key blocks, sfb_build_stream +
sfb_fused_attention_streamed) against the CPU oracle and against the scheduled entry point."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, qkv, rel_err
from sfb import sfb

pytestmark = pytest.mark.gpu
THREADS = 16


def run_streamed(Q, K, V, nn_lut, nb, bs, blocks, scale, bf16, level=True, lut_heads=1, mask=None, valid_len=None,
                 mask_heads=1, wg_slots=None, out_bf16=False, want_lse=False, launches=2):
    B, L, H, d = Q.shape
    masked = mask is not None or valid_len is not None or want_lse
    stream = sfb.build_stream(nn_lut, nb, B, H, bs, lut_heads=lut_heads, wg_slots=wg_slots, level=level, d=d,
                              bf16=bf16, masked=masked)
    ws = torch.zeros(sfb.stream_workspace_bytes(stream, d), dtype=torch.uint8, device="cuda")
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    nn, blob = sfb.to_device(nn_lut), sfb.to_device(stream["blob"])
    m = None if mask is None else sfb.to_device(mask)
    vl = None if valid_len is None else sfb.to_device(np.asarray(valid_len, np.int32))
    outs = []
    for _ in range(launches):   # later launches find the flags as the first one left them
        out = torch.full((B, L, H, d), 7.0, device="cuda", dtype=torch.bfloat16 if out_bf16 else torch.float32)
        lse = torch.full((B, H, L), 7.0, device="cuda") if want_lse else None
        sfb.fused_attention_streamed(q, k, v, nn, blob, stream, ws, bs, blocks, scale, mask=m, valid_len=vl,
                                     mask_heads=mask_heads, out=out, lse=lse)
        torch.cuda.synchronize()
        outs.append(out)
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    assert sfb.stream_status(stream, d, ws) == 0
    assert int(ws[:max(4 * stream["plan"].n_parts, 4)].view(torch.int32).abs().sum()) == 0, "flags must be left at zero"
    return (outs[0], lse, stream) if want_lse else (outs[0], stream)


@pytest.mark.parametrize("level", [True, False])
@pytest.mark.parametrize("bf16", [True, False])
def test_c4_bigbird_streamed(bf16, level):
    B, H, L, d, bs = 4, 12, 4096, 64, 64
    luts = sfb.build_luts(PATTERNS["bigbird"](L // bs))
    Q, K, V = qkv(B, L, H, d, seed=404, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    got, stream = run_streamed(Q, K, V, luts["nn_lut"], L // bs, bs, luts["blocks"], 0.125, bf16, level=level)
    got = got.cpu().numpy()
    assert stream["plan"].n_parts > 0
    diff = np.abs(got.astype(np.float64) - want).max(axis=(1, 3)) / np.abs(want).max(axis=(1, 3))
    print("partial records", stream["plan"].n_parts, "balance %.3f" % stream["plan"].balance,
          "worst (batch, head) error %.3e" % diff.max(), flush=True)
    assert np.isfinite(got).all() and diff.max() <= (TOL_BF16 if bf16 else TOL_F32)


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("level,wg_slots", [(True, 16), (False, 1024), (True, 7), (False, 64), (True, 256)])
def test_streamed_masks_padding_split_rows(bf16, level, wg_slots):
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
    got, _ = run_streamed(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, bf16, level=level,
                          mask=mask, valid_len=valid, wg_slots=wg_slots)
    assert rel_err(got.cpu().numpy(), want) <= tol
    assert (got[:, 5 * bs:6 * bs] == 0).all()
    # the same layout without mask and padding takes the kernels' other instantiation
    plain = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    got, _ = run_streamed(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, bf16, level=level,
                          wg_slots=wg_slots)
    assert rel_err(got.cpu().numpy(), plain) <= tol


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("bs", [32, 64])
def test_streamed_per_head_luts_and_masks(bf16, bs):
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
    for level, wg_slots in ((True, 40), (False, 40), (True, 256)):
        got, stream = run_streamed(Q, K, V, nn, nb, bs, blocks, 0.125, bf16, level=level, lut_heads=H,
                                   mask=masks, mask_heads=H, wg_slots=wg_slots)
        assert stream["plan"].n_blocks == B * H * blocks
        assert rel_err(got.cpu().numpy(), want) <= (TOL_BF16 if bf16 else TOL_F32)
    # without masks: the loop that keeps one offset per item, over per-head streams
    want = orc.attention(Q, K, V, nn, bs, 0.125, lut_heads=H, blocks=blocks, nthreads=THREADS)
    got, _ = run_streamed(Q, K, V, nn, nb, bs, blocks, 0.125, bf16, lut_heads=H, wg_slots=40)
    assert rel_err(got.cpu().numpy(), want) <= (TOL_BF16 if bf16 else TOL_F32)


def test_streamed_bf16_output_and_lse_match_the_scheduled_entry():
    bs, nb, B, H, d = 64, 32, 2, 4, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    Q, K, V = qkv(B, L, H, d, seed=77, bf16=True)
    got, lse, _ = run_streamed(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, True, wg_slots=64,
                               out_bf16=True, want_lse=True)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    sched = sfb.build_schedule(luts["nn_lut"], nb, 8)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    o32, lse2 = sfb.fused_attention_forward_lse(q, k, v, sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"]),
                                                sched, ws, bs, luts["blocks"], 0.125)
    torch.cuda.synchronize()
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    assert rel_err(got.float().cpu().numpy(), want) <= TOL_BF16
    # the same arithmetic; rows may be cut at other places
    assert rel_err(got.float().cpu().numpy(), o32.cpu().numpy()) <= 2.0 ** -7
    assert torch.allclose(lse, lse2, rtol=0, atol=1e-3)


def test_streamed_overflowing_scores_take_the_general_loop():
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
    for wg_slots in (8, 3, 40):   # whole rows one after the other in a stream; cut rows
        got, _ = run_streamed(Q, K, V, luts["nn_lut"], nb, bs, luts["blocks"], 0.125, True, wg_slots=wg_slots)
        got = got.cpu().numpy()
        assert np.isfinite(got).all()
        assert rel_err(got, want) <= TOL_BF16

    # the unscheduled and the scheduled entry points run the same loops
    from gpu_common import run_fused
    assert rel_err(run_fused(Q, K, V, luts, bs, 0.125, bf16=True), want) <= TOL_BF16
    assert rel_err(run_fused(Q, K, V, luts, bs, 0.125, bf16=True, max_blocks=3), want) <= TOL_BF16


@pytest.mark.needs_device
def test_a_merge_whose_record_never_arrives_gives_up_and_the_workspace_recovers():
    """Failure handling, forced from the host: in the plan's copy on the device the merge of the last records expects
    one record more than exist (its flag, in the padding of the flag area, is never set).  The merge's wait is
    bounded (about a second), so the launch ends normally with status 1 and every other row right; the binding then
    clears the workspace (sfb_stream_reset) and the next launch, with the plan as built, is right and reports 0."""
    bs, nb, B, H, d = 64, 16, 2, 3, 64
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    Q, K, V = qkv(B, nb * bs, H, d, seed=515, bf16=True)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    nn = sfb.to_device(luts["nn_lut"])
    stream = sfb.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=61)
    n_parts = stream["plan"].n_parts
    assert n_parts > 0 and (4 * n_parts) % 256 != 0, "the flag area has padding after the last flag"
    ws = torch.zeros(sfb.stream_workspace_bytes(stream, d), dtype=torch.uint8, device="cuda")
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    good = stream["blob"].copy()
    merges = stream["merges"]   # a view of stream["blob"]
    last = int(np.argmax(merges["part"] + merges["nparts"]))
    assert merges["part"][last] + merges["nparts"][last] == n_parts
    merges["nparts"][last] += 1
    b, h, r = int(merges["batch"][last]), int(merges["head"][last]), int(merges["row"][last])
    out = torch.full((B, nb * bs, H, d), 7.0, device="cuda")
    sfb.fused_attention_streamed(q, k, v, nn, sfb.to_device(stream["blob"]), stream, ws, bs, luts["blocks"], 0.125, out=out)
    torch.cuda.synchronize()
    assert sfb.stream_status(stream, d, ws) == 1
    got = out.cpu().numpy()
    assert (got[b, r * bs:(r + 1) * bs, h] == 7.0).all()
    got[b, r * bs:(r + 1) * bs, h] = want[b, r * bs:(r + 1) * bs, h]
    assert rel_err(got, want) <= TOL_BF16
    for _ in range(2):
        out = sfb.fused_attention_streamed(q, k, v, nn, sfb.to_device(good), stream, ws, bs, luts["blocks"], 0.125)
        torch.cuda.synchronize()
        assert sfb.stream_status(stream, d, ws) == 0
        assert rel_err(out.cpu().numpy(), want) <= TOL_BF16
