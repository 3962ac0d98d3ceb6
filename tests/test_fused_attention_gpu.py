"""Parity of the fused HIP attention (through the C ABI) against the CPU oracle, on the workload
configurations and on edge cases; bit-level properties at full size."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, elementwise_err, qkv, rel_err, run_fused
from sfb import sfb

pytestmark = pytest.mark.gpu
THREADS = 16


def check(got, want, tol):
    err = rel_err(got, want)
    # the gate is max|diff| / max|want|; the element-wise figure (denominator floored at 10% of the
    # largest magnitude) is reported and bounded loosely
    ew = elementwise_err(got, want, floor=1e-1 * np.abs(want).max())
    print("rel_err %.3e elementwise(floor 10%% of max) %.3e" % (err, ew), flush=True)
    assert np.isfinite(got).all()
    assert err <= tol, err
    assert ew <= 10 * tol, ew


def test_c1_local_fp32():
    B, H, L, d, bs = 1, 12, 512, 64, 32
    luts = sfb.build_luts(PATTERNS["local"](L // bs))
    assert luts["blocks"] == 46
    Q, K, V = qkv(B, L, H, d, seed=1)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    check(run_fused(Q, K, V, luts, bs, 0.125), want, TOL_F32)


def test_c2_fixed_padding_fp32():
    B, H, L, d, bs = 8, 12, 1024, 64, 32
    luts = sfb.build_luts(PATTERNS["fixed"](L // bs))
    assert luts["blocks"] == 352
    Q, K, V = qkv(B, L, H, d, seed=2)
    valid = orc.fill_uniform_int((B,), 22, 768, 1024)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, valid_len=valid, nthreads=THREADS)
    check(run_fused(Q, K, V, luts, bs, 0.125, valid_len=valid), want, TOL_F32)


@pytest.mark.parametrize("bf16", [False, True])
def test_c3_strided(bf16):
    B, H, L, d, bs = 2, 12, 2048, 64, 64  # batch 2 of the configuration's 8: the oracle stays in seconds
    luts = sfb.build_luts(PATTERNS["strided"](L // bs))
    assert luts["blocks"] == 346
    Q, K, V = qkv(B, L, H, d, seed=3, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    check(run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16), want, TOL_BF16 if bf16 else TOL_F32)


@pytest.mark.parametrize("bf16", [True, False])
def test_c4_bigbird(bf16):
    B, H, L, d, bs = 1, 3, 4096, 64, 64  # 3 of the 48 (batch, head) pairs against the oracle
    luts = sfb.build_luts(PATTERNS["bigbird"](L // bs))
    assert luts["blocks"] == 622 and luts["nn_max"] == 64
    Q, K, V = qkv(B, L, H, d, seed=4, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    check(run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16), want, TOL_BF16 if bf16 else TOL_F32)


def test_c4_full_size_properties():
    """B4 H12 L4096: closed form on all-ones inputs, batch/head independence, fp32 vs bf16 kernels."""
    B, H, L, d, bs = 4, 12, 4096, 64, 64
    lay = PATTERNS["bigbird"](L // bs)
    luts = sfb.build_luts(lay)
    ones = np.ones((B, L, H, d), np.float32)
    for bf16 in (True, False):
        O = run_fused(ones, ones, ones, luts, bs, 0.125, bf16=bf16)
        n_keys = (lay.sum(axis=1) * bs).astype(np.float32)
        want = np.repeat(n_keys / (n_keys + np.float32(1e-6)), bs)[None, :, None, None]
        assert np.abs(O - want).max() <= 1e-6
    Q, K, V = qkv(1, L, 2, d, seed=44, bf16=True)
    tile = lambda x: np.ascontiguousarray(np.tile(x, (B, 1, H // 2, 1)))
    Ob = run_fused(tile(Q), tile(K), tile(V), luts, bs, 0.125, bf16=True)
    assert np.array_equal(Ob, np.tile(Ob[:1, :, :2], (B, 1, H // 2, 1)))  # every (b,h) copy identical
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    check(Ob[:1, :, :2], want, TOL_BF16)
    Of = run_fused(tile(Q), tile(K), tile(V), luts, bs, 0.125, bf16=False)
    check(Of[:1, :, :2], want, TOL_F32)


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("pattern", ["causal", "local_causal", "bigbird", "full"])
def test_masks_and_padding(pattern, bs, bf16):
    nb, B, H, d = 8, 3, 2, 64
    L = nb * bs
    luts = sfb.build_luts(PATTERNS[pattern](nb))
    kind = {"causal": sfb.MASK_CAUSAL_DIAG, "local_causal": sfb.MASK_LOCAL}.get(pattern, sfb.MASK_ALL)
    mask = sfb.pack_mask(sfb.element_mask(luts["nt_lut"], bs, kind, local_attn_ctx=bs)) if kind else None
    if pattern == "full":  # a random element mask, so every bit position is exercised
        keep = (np.random.default_rng(bs).random((luts["blocks"], bs, bs)) < 0.7).astype(np.uint8)
        mask = sfb.pack_mask(keep)
    valid = np.array([L, L - bs - 7, 5], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=50 + bs, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, mask=mask, valid_len=valid, nthreads=THREADS)
    got = run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16, mask=mask, valid_len=valid)
    check(got, want, TOL_BF16 if bf16 else TOL_F32)
    # same result without the launch-order table
    got2 = run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16, mask=mask, valid_len=valid, use_order=False)
    assert np.array_equal(got, got2)


@pytest.mark.parametrize("bf16", [False, True])
def test_empty_rows_and_fully_masked_rows(bf16):
    bs, nb, B, H, d = 32, 6, 2, 3, 64
    L = bs * nb
    lay = PATTERNS["local"](nb).copy()
    lay[2] = 0
    luts = sfb.build_luts(lay)
    Q, K, V = qkv(B, L, H, d, seed=70, bf16=bf16)
    valid = np.array([L, 0], np.int32)
    got = run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16, valid_len=valid)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, valid_len=valid)
    assert (got[:, 2 * bs:3 * bs] == 0).all() and (got[1] == 0).all()
    check(got, want, TOL_BF16 if bf16 else TOL_F32)


def test_per_head_luts_and_masks():
    bs, nb, B, H, d = 32, 8, 2, 4, 64
    L = bs * nb
    lay = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lay[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    assert all(p["blocks"] == blocks for p in per_head)
    nn = np.concatenate([p["nn_lut"] for p in per_head])
    masks = np.concatenate([sfb.pack_mask(sfb.element_mask(p["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG))
                            for p in per_head])
    Q, K, V = qkv(B, L, H, d, seed=80)
    want = orc.attention(Q, K, V, nn, bs, 0.125, mask=masks, lut_heads=H, mask_heads=H, blocks=blocks)
    got = run_fused(Q, K, V, per_head[0], bs, 0.125, mask=masks, lut_heads=H, mask_heads=H, nn_lut=nn,
                    blocks=blocks, use_order=False)
    check(got, want, TOL_F32)


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("max_blocks", [8, 3, 1])
def test_scheduled_split_rows(bf16, max_blocks):
    """Rows cut into chunks whose partials are merged by the last chunk to finish: same result as the
    oracle, masks and padding included, and the workspace is reusable launch after launch."""
    bs, nb, B, H, d = 64, 16, 2, 3, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    keep = (np.random.default_rng(7).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    mask = sfb.pack_mask(keep)
    valid = np.array([L, L - 100], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=95, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, mask=mask, valid_len=valid, nthreads=THREADS)
    sched = sfb.build_schedule(luts["nn_lut"], nb, max_blocks)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    for _ in range(3):
        got = run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16, mask=mask, valid_len=valid,
                        max_blocks=max_blocks, workspace=ws)
        check(got, want, TOL_BF16 if bf16 else TOL_F32)


def test_c4_scheduled_full_size():
    B, H, L, d, bs = 4, 12, 4096, 64, 64
    luts = sfb.build_luts(PATTERNS["bigbird"](L // bs))
    Q, K, V = qkv(1, L, 2, d, seed=44, bf16=True)
    tile = lambda x: np.ascontiguousarray(np.tile(x, (B, 1, H // 2, 1)))
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    got = run_fused(tile(Q), tile(K), tile(V), luts, bs, 0.125, bf16=True, max_blocks=8)
    for b in range(B):
        for h in range(0, H, 2):
            assert rel_err(got[b:b + 1, :, h:h + 2], want) <= TOL_BF16
    plain = run_fused(tile(Q), tile(K), tile(V), luts, bs, 0.125, bf16=True)
    unsplit = [r for r in range(L // bs) if luts["nn_lut"][r, 1] <= 8]
    rows = np.concatenate([np.arange(r * bs, (r + 1) * bs) for r in unsplit])
    assert np.array_equal(got[:, rows], plain[:, rows])  # unsplit rows take the identical code path
    assert rel_err(got, plain) <= 5e-3  # split rows: probabilities are rounded to bf16 relative to per-chunk maxima


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("scheduled", [False, True])
def test_rows_longer_than_64_key_blocks(bf16, scheduled):
    """Dense layout with 80 key blocks per row: a work-group walks more LUT entries than one wave holds
    (the bf16 kernel keeps 64 entries in registers and fetches the next window on the way)."""
    bs, nb, B, H, d = 64, 80, 1, 2, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["full"](nb))
    valid = np.array([L - 37], np.int32)
    Q, K, V = qkv(B, L, H, d, seed=131, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, valid_len=valid, nthreads=THREADS)
    got = run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16, valid_len=valid, max_blocks=1000 if scheduled else None)
    check(got, want, TOL_BF16 if bf16 else TOL_F32)
    got = run_fused(Q, K, V, luts, bs, 0.125, bf16=bf16, max_blocks=1000 if scheduled else None)
    check(got, orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS), TOL_BF16 if bf16 else TOL_F32)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("d", [32, 96, 128])
@pytest.mark.parametrize("bs", [32, 64])
def test_head_sizes_other_than_64(d, bs, bf16):
    """Head size 32, 96 or 128 (the reference's K64 = false paths), fp32 and bf16 tensors: fused kernel, plain,
    scheduled with split rows and streamed, masked and padded."""
    nb, B, H = 16, 2, 3
    tol = TOL_BF16 if bf16 else TOL_F32
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    keep = (np.random.default_rng(d).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    mask = sfb.pack_mask(keep)
    valid = np.array([nb * bs, nb * bs - bs - 5], np.int32)
    Q, K, V = qkv(B, nb * bs, H, d, seed=d + bs, bf16=bf16)
    scale = float(1.0 / np.sqrt(d))
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, mask=mask, valid_len=valid, nthreads=THREADS)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16, mask=mask, valid_len=valid), want, tol)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16, mask=mask, valid_len=valid, max_blocks=3), want, tol)
    plain = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, nthreads=THREADS)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16), plain, tol)
    check(run_fused(Q, K, V, luts, bs, scale, bf16=bf16, max_blocks=3), plain, tol)
    # streamed launches: rows cut into chunks, merged from partial records
    stream = sfb.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=64)
    assert stream["plan"].n_parts > 0
    ws = torch.zeros(sfb.stream_workspace_bytes(stream, d), dtype=torch.uint8, device="cuda")
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    nn, blob = sfb.to_device(luts["nn_lut"]), sfb.to_device(stream["blob"])
    for m, vl, ref in ((None, None, plain), (sfb.to_device(mask), sfb.to_device(valid), want)):
        out = sfb.fused_attention_streamed(q, k, v, nn, blob, stream, ws, bs, luts["blocks"], scale, mask=m, valid_len=vl)
        torch.cuda.synchronize()
        assert sfb.stream_status(stream, d, ws) == 0
        check(out.cpu().numpy(), ref, tol)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("d", [64, 32])
def test_token_stride_of_a_merged_projection(bf16, d):
    """Q, K and V as column slices of one [B, L, 3 H d] tensor (sfb_fused_attention_scheduled_strided): the same
    bits as the launch on three dense tensors, split rows, mask and padding included."""
    bs, nb, B, H = 64, 16, 2, 3
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    keep = (np.random.default_rng(7).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    mask = sfb.to_device(sfb.pack_mask(keep))
    valid = sfb.to_device(np.array([nb * bs, nb * bs - bs - 5], np.int32))
    Q, K, V = qkv(B, nb * bs, H, d, seed=91 + d, bf16=bf16)
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    merged = torch.cat([t.reshape(B, nb * bs, H * d) for t in (q, k, v)], dim=2).contiguous()
    sched = sfb.build_schedule(luts["nn_lut"], nb, 3)
    assert sched["n_parts"] > 0
    nn, items = sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"])
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    scale = float(1.0 / np.sqrt(d))
    for m, vl in ((None, None), (mask, valid)):
        for out_dtype in (sfb.F32, sfb.BF16):
            dense = sfb.fused_attention_scheduled(q, k, v, nn, items, sched, ws, bs, luts["blocks"], scale, mask=m,
                                                  valid_len=vl, out_dtype=out_dtype)
            strided = sfb.fused_attention_scheduled_strided(merged, nn, items, sched, ws, bs, luts["blocks"], scale, H,
                                                            mask=m, valid_len=vl, out_dtype=out_dtype)
            torch.cuda.synchronize()
            assert torch.equal(dense, strided)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, nthreads=THREADS)
    got = sfb.fused_attention_scheduled_strided(merged, nn, items, sched, ws, bs, luts["blocks"], scale, H)
    check(got.cpu().numpy(), want, TOL_BF16 if bf16 else TOL_F32)
    with pytest.raises(sfb.SfbError) as e:   # a stride that is not a multiple of 16 bytes
        bad = torch.zeros((B, nb * bs, 3 * H * d + 3), device="cuda", dtype=merged.dtype)
        lib_call = sfb.lib.sfb_fused_attention_scheduled_strided
        sfb.capi._check(lib_call(None, C.c_void_p(bad.data_ptr()), C.c_void_p(bad.data_ptr()), C.c_void_p(bad.data_ptr()),
                                 C.c_void_p(got.data_ptr()), sfb.BF16 if bf16 else sfb.F32, sfb.F32, C.c_void_p(nn.data_ptr()),
                                 None, None, C.c_void_p(items.data_ptr()), C.c_uint32(sched["n_items"]),
                                 C.c_uint32(sched["n_heavy"]), C.c_uint32(sched["n_slots"]), C.c_uint32(sched["n_parts"]),
                                 C.c_void_p(ws.data_ptr()), C.c_size_t(ws.numel()), C.c_uint32(bs),
                                 C.c_uint32(luts["blocks"]), C.c_uint32(B), C.c_uint32(nb), C.c_uint32(H), C.c_uint32(d),
                                 C.c_uint32(3 * H * d + 3), C.c_uint32(1), C.c_float(scale)), "strided")
    assert e.value.status == 4


def test_head_size_errors():
    luts = sfb.build_luts(PATTERNS["full"](1))
    # head sizes: multiples of the 16-byte vector (8 bf16, 4 floats) up to 128
    for dtype, d in ((torch.bfloat16, 132), (torch.float32, 132), (torch.bfloat16, 84), (torch.float32, 42)):
        q = torch.zeros((1, 64, 1, d), device="cuda", dtype=dtype)
        with pytest.raises(sfb.SfbError) as e:
            sfb.fused_attention(q, q, q, sfb.to_device(luts["nn_lut"]), 64, 1, 0.125)
        assert e.value.status == 3


@pytest.mark.parametrize("bf16_in", [False, True])
@pytest.mark.parametrize("bs,max_blocks", [(64, 4), (32, 100)])
def test_bf16_output_is_the_fp32_output_rounded_once(bs, max_blocks, bf16_in):
    """sfb_fused_attention_scheduled_to with bf16 output (split rows merged and rows kept whole, zero rows too)."""
    nb, B, H, d = 16, 2, 3, 64
    lay = PATTERNS["bigbird"](nb).copy()
    lay[5] = 0
    luts = sfb.build_luts(lay)
    Q, K, V = qkv(B, nb * bs, H, d, seed=77, bf16=bf16_in)
    q, k, v = (dev(x, bf16_in) for x in (Q, K, V))
    sched = sfb.build_schedule(luts["nn_lut"], nb, max_blocks)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    args = (q, k, v, sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"]), sched, ws, bs, luts["blocks"], 0.125)
    o32 = sfb.fused_attention_scheduled(*args)
    o16 = torch.full((B, nb * bs, H, d), 7.0, device="cuda", dtype=torch.bfloat16)
    sfb.fused_attention_scheduled(*args, out=o16)
    torch.cuda.synchronize()
    assert torch.equal(o16, o32.to(torch.bfloat16))
    assert (o16[:, 5 * bs:6 * bs] == 0).all()
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125)
    assert rel_err(o16.float().cpu().numpy(), want) <= TOL_BF16


@pytest.mark.needs_device
def test_scheduled_launch_in_a_hip_graph():
    """The scheduled launch (split rows, counters reset by the kernel itself, no memset) captured into a graph:
    every replay, with eager launches and synchronisations in between, gives the eager result bit for bit."""
    bs, nb, B, H, d = 64, 32, 2, 4, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    Q, K, V = qkv(B, L, H, d, seed=77, bf16=True)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    nn = sfb.to_device(luts["nn_lut"])
    sched = sfb.build_schedule(luts["nn_lut"], nb, 8)
    items = sfb.to_device(sched["items"])
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    launch = lambda out: sfb.fused_attention_scheduled(q, k, v, nn, items, sched, ws, bs, luts["blocks"], 0.125, out=out)
    eager = torch.empty((B, L, H, d), dtype=torch.float32, device="cuda")
    launch(eager)
    torch.cuda.synchronize()
    captured = torch.zeros_like(eager)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(captured)   # warm-up on the capture stream
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            launch(captured)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        captured.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager)
        other = torch.empty_like(eager)
        launch(other)   # eager launch on the same workspace between replays
        torch.cuda.synchronize()
        assert torch.equal(other, eager)


def test_scale_and_large_scores():
    # scores far from zero: the running maximum and the 1e-6 term must still follow the oracle
    bs, nb, B, H, d = 64, 4, 1, 2, 64
    L = bs * nb
    luts = sfb.build_luts(PATTERNS["full"](nb))
    Q, K, V = qkv(B, L, H, d, seed=90)
    Q *= 6.0
    for scale in (0.125, 1.0, 0.01):
        want = orc.attention(Q, K, V, luts["nn_lut"], bs, scale)
        check(run_fused(Q, K, V, luts, bs, scale), want, TOL_F32)


def test_argument_errors():
    q = torch.zeros((1, 64, 1, 64), device="cuda")
    lut = sfb.to_device(np.zeros((3, 2), np.uint32))
    call = lambda **kw: sfb.lib.sfb_fused_attention(
        None, kw.get("q", C.c_void_p(q.data_ptr())), C.c_void_p(q.data_ptr()), C.c_void_p(q.data_ptr()),
        C.c_void_p(q.data_ptr()), kw.get("dtype", 0), C.c_void_p(lut.data_ptr()), None, None, None,
        C.c_uint32(kw.get("bs", 64)), C.c_uint32(1), C.c_uint32(1), C.c_uint32(1), C.c_uint32(1),
        C.c_uint32(kw.get("d", 64)), C.c_uint32(1), C.c_uint32(2), C.c_uint32(1), C.c_float(0.125))
    assert call(q=None) == 1
    assert call(bs=16) == 2
    assert call(d=50) == 3      # fp32 rows are whole 16-byte vectors: multiples of 4
    assert call(d=132) == 3
    assert call(d=44, dtype=1) == 3   # bf16: multiples of 8
    assert call(dtype=7) == 5
    assert call(q=C.c_void_p(q.data_ptr() + 4)) == 6
