"""The workload configurations at their full sizes, with independent data for every (batch, head), through the
launches the benchmark times: every output element is compared with the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, qkv, rel_err
from sfb import sfb
from test_layer_gpu import T, layer_weights

pytestmark = pytest.mark.gpu
THREADS = 16


def scheduled(Q, K, V, luts, bs, scale, bf16, max_blocks):
    B, L, H, d = Q.shape
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    sched = sfb.build_schedule(luts["nn_lut"], L // bs, max_blocks)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    nn, items = sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"])
    outs = []
    for _ in range(2):   # the second launch finds the arrival counters as the first one left them
        outs.append(sfb.fused_attention_scheduled(q, k, v, nn, items, sched, ws, bs, luts["blocks"], scale).cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    return outs[0], sched


def per_head_errors(got, want):
    """max |diff| / max |want| of every (batch, head) slice: a batch / head mix-up shows as an error near 1."""
    diff = np.abs(got.astype(np.float64) - want).max(axis=(1, 3))
    return diff / np.abs(want).max(axis=(1, 3))


@pytest.mark.parametrize("bf16", [True, False])
def test_c4_bigbird_as_benchmarked(bf16):
    """B4 H12 L4096 d64 block 64, the chunk length sfb_suggest_max_blocks picks for 48 (batch, head) pairs."""
    B, H, L, d, bs = 4, 12, 4096, 64, 64
    luts = sfb.build_luts(PATTERNS["bigbird"](L // bs))
    assert luts["blocks"] == 622
    max_blocks = sfb.suggest_max_blocks(luts["nn_lut"], L // bs, B * H)
    Q, K, V = qkv(B, L, H, d, seed=404, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    got, sched = scheduled(Q, K, V, luts, bs, 0.125, bf16, max_blocks)
    assert sched["n_heavy"] > 0 and sched["n_parts"] > 0   # split global rows, issued first for all heads
    errs = per_head_errors(got, want)
    print("max_blocks", max_blocks, "worst (batch, head) error %.3e" % errs.max(), flush=True)
    assert np.isfinite(got).all()
    assert errs.max() <= (TOL_BF16 if bf16 else TOL_F32)


def test_c4_unfused_trio_full_size():
    """The unfused sdd -> softmax -> dsd sequence and the two-stage fusion at the benchmarked size (bf16 tensors, bf16
    S and P): the output against the oracle per (batch, head), the two ways to P against each other, and every
    stage bit-identical over repeated launches (the streaming kernels wait on counts of loads and stores in
    flight; a count that is too generous would show here as a difference between launches)."""
    B, H, L, d, bs = 4, 12, 4096, 64, 64
    nb = L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    blocks = luts["blocks"]
    Q, K, V = qkv(B, L, H, d, seed=405, bf16=True)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    nt, nn = sfb.to_device(luts["nt_lut"]), sfb.to_device(luts["nn_lut"])
    runs = []
    for _ in range(3):
        S = sfb.bst_sgemm_nt(nt, q, k, bs, blocks, out_dtype=sfb.BF16)
        P = sfb.BlocksparseMaskedSoftmax(nn, None, S, nb, 0.125)
        O = sfb.bst_sgemm_xn(nn, P, v, nb)
        P2 = sfb.fusion_attention2(nn, q, k, bs, blocks, 0.125, out_dtype=sfb.BF16,
                                   row_order=sfb.to_device(luts["row_order"]))
        torch.cuda.synchronize()
        runs.append((S, P, O, P2))
    for later in runs[1:]:
        for a, b in zip(runs[0], later):
            assert torch.equal(a, b)
    S, P, O, P2 = runs[0]
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    errs = per_head_errors(O.cpu().numpy(), want)
    print("worst (batch, head) error %.3e" % errs.max(), flush=True)
    # S and P go through memory as bf16: two roundings more than the fused kernel's output carries (each stage
    # alone is held to TOL_BF16 against the oracle in test_unfused_gpu.py); a (batch, head) mix-up would be near 1
    assert errs.max() <= 2 * TOL_BF16
    # P from bf16-rounded scores against P from the fused product's fp32 scores: the rounding of S moves a
    # probability by at most |s| * 2^-9 * scale relative
    diff = (P.float() - P2.float()).abs().amax(dim=(2, 3, 4)) / P2.float().amax(dim=(2, 3, 4))
    assert float(diff.max()) <= 3e-2
    rows = P2.float().sum(dim=-1)   # every query row of every block: the blocks of a row add up to 1
    total = torch.zeros((B, H, nb, bs), device="cuda")
    total.index_add_(2, torch.from_numpy(luts["nt_lut"][:, 0].astype(np.int64)).cuda(), rows)
    assert float((total - 1).abs().max()) <= 2e-2


@pytest.mark.parametrize("bf16", [True, False])
def test_c3_strided_full_batch(bf16):
    B, H, L, d, bs = 8, 12, 2048, 64, 64
    luts = sfb.build_luts(PATTERNS["strided"](L // bs))
    assert luts["blocks"] == 346
    Q, K, V = qkv(B, L, H, d, seed=303, bf16=bf16)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, nthreads=THREADS)
    tol = TOL_BF16 if bf16 else TOL_F32
    got, _ = scheduled(Q, K, V, luts, bs, 0.125, bf16, sfb.suggest_max_blocks(luts["nn_lut"], L // bs, B * H))
    assert per_head_errors(got, want).max() <= tol
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    plain = sfb.fused_attention(q, k, v, sfb.to_device(luts["nn_lut"]), bs, luts["blocks"], 0.125,
                                row_order=sfb.to_device(luts["row_order"])).cpu().numpy()
    assert per_head_errors(plain, want).max() <= tol


@pytest.mark.parametrize("bf16", [True, False])
def test_c5_encoder_layer_full_size(bf16):
    """B8 L4096, hidden 768, 12 heads, FFN 3072, BigBird attention; input = token embedding (30522-entry table,
    ids uniform over it) + learned positions, through sfb_embedding_lookup and sfb_encoder_layer_forward with
    the chunk length the benchmark's layer uses."""
    B, L, H, d, ffn, bs, vocab = 8, 4096, 12, 64, 3072, 64, 30522
    n, nb = H * d, L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    w = layer_weights(n, ffn, 500)
    tok = orc.fill_normal((vocab, n), 601, 0.02)
    pos = orc.fill_normal((L, n), 602, 0.02)
    ids = orc.fill_uniform_int((B, L), 603, 0, vocab - 1)
    assert ids.min() >= 0 and ids.max() < vocab and len(np.unique(ids)) > 10000
    x_want = (tok[ids] + pos[None]).reshape(B * L, n)   # embedding.h:5-12 then ewops.h:276-282: one fp32 add
    x = sfb.embedding_lookup(T(tok), T(ids), T(pos)).reshape(B * L, n)
    assert np.array_equal(x.cpu().numpy(), x_want)
    max_blocks = sfb.suggest_max_blocks(luts["nn_lut"], nb, B * H)
    layer = sfb.EncoderLayer({k: T(v) for k, v in w.items()}, luts, bs, H, d, ffn,
                             dtype=sfb.BF16 if bf16 else sfb.F32, max_blocks=max_blocks)
    got = layer.forward(x, B, L).cpu().numpy()
    torch.cuda.synchronize()
    want = orc.encoder_layer(x_want, w, luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"], operands_bf16=bf16,
                             nthreads=THREADS)
    assert np.isfinite(got).all()
    # per sequence, so that a sequence taking another one's rows cannot hide behind the rest
    errs = [rel_err(got[b * L:(b + 1) * L], want[b * L:(b + 1) * L]) for b in range(B)]
    print("max_blocks", max_blocks, "per-sequence errors", ["%.2e" % e for e in errs], flush=True)
    assert max(errs) <= (1e-2 if bf16 else 1e-4)
