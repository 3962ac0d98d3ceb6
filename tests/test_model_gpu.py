"""Whole-model forward (embedding, N encoder layers, tied logits, cross-entropy loss) and its new pieces against
the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, rel_err
from sfb import sfb
from test_oracle_model import make_model

pytestmark = pytest.mark.gpu
T = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("rows,vocab", [(64, 256), (33, 30522), (5, 7)])
def test_cross_entropy_matches_oracle(rows, vocab):
    logits = orc.fill_normal((rows, vocab), 3) * 3
    labels = orc.fill_uniform_int((rows,), 4, 0, vocab - 1)
    want, want_rows, want_d = orc.softmax_cross_entropy(logits, labels, want_grad=True)
    loss, row_loss, d = sfb.softmax_cross_entropy(T(logits), T(labels), want_grad=True)
    assert rel_err(row_loss.cpu().numpy(), want_rows) <= 1e-5
    assert abs(float(loss) - want) <= 1e-5 * want
    assert rel_err(d.cpu().numpy(), want_d) <= 1e-4   # the reference sums 30522 floats one by one
    # in place, and the same bits on every call
    buf = T(logits)
    loss2, _, d2 = sfb.softmax_cross_entropy(buf, T(labels), want_grad=True, in_place=True)
    assert d2.data_ptr() == buf.data_ptr() and torch.equal(d2, d) and torch.equal(loss2, loss)


def test_cross_entropy_label_outside_the_vocabulary_selects_nothing():
    logits = orc.fill_normal((4, 50), 5)
    labels = np.array([3, -1, 50, 49], np.int32)
    loss, row_loss, d = sfb.softmax_cross_entropy(T(logits), T(labels), want_grad=True)
    rows = row_loss.cpu().numpy()
    assert rows[1] == 0 and rows[2] == 0 and rows[0] > 0 and rows[3] > 0
    assert abs(float(loss) - rows.sum() / 4) <= 1e-6
    assert np.allclose(d.cpu().numpy()[1].sum(), 1.0, atol=1e-5)   # plain softmax, nothing subtracted


@pytest.mark.parametrize("bf16", [False, True])
def test_gemm_nt_matches_oracle(bf16):
    m, k, n = 200, 768, 1000
    A = orc.fill_normal((m, k), 9)
    W = orc.fill_normal((n, k), 10, 0.02)
    if bf16:
        A, W = orc.round_bf16(A), orc.round_bf16(W)
    a, w = T(A), T(W)
    if bf16:
        a, w = a.to(torch.bfloat16), w.to(torch.bfloat16)
    got = sfb.gemm_nt(a, w).cpu().numpy()
    assert rel_err(got, orc.sgemm_nt(A, W, nthreads=16)) <= 1e-5
    assert rel_err(got, A.astype(np.float64) @ W.astype(np.float64).T) <= 1e-5


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("max_blocks", [0, 4])
def test_pre_ln_layer_matches_oracle(bf16, max_blocks):
    B, L, H, d, ffn, bs = 2, 512, 4, 64, 1024, 64
    n, nb = H * d, L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    layers, _, _ = make_model(1, n, ffn, 10, L, seed=500)
    x = orc.fill_normal((B * L, n), 501)
    want = orc.encoder_layer_pre_ln(x, layers[0], luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"],
                                    operands_bf16=bf16, nthreads=16)
    layer = sfb.EncoderLayer({k: T(v) for k, v in layers[0].items()}, luts, bs, H, d, ffn,
                             dtype=sfb.BF16 if bf16 else sfb.F32, max_blocks=max_blocks, pre_ln=True)
    got = layer.forward(T(x), B, L).cpu().numpy()
    assert rel_err(got, want) <= (1e-2 if bf16 else 1e-4)
    post = orc.encoder_layer(x, layers[0], luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"], nthreads=16)
    assert rel_err(got, post) > 0.05   # the two wirings are not confused


@pytest.mark.parametrize("pre_ln", [True, False])
@pytest.mark.parametrize("bf16", [False, True])
def test_model_forward_matches_oracle(bf16, pre_ln):
    B, L, H, d, ffn, bs, vocab, n_layers = 2, 512, 4, 64, 1024, 64, 256, 3
    n, nb = H * d, L // bs
    luts = sfb.build_luts(PATTERNS["causal"](nb))
    mask = sfb.pack_mask(sfb.element_mask(luts["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG))
    valid = np.array([L, L - 70], np.int32)
    # small embeddings keep the logits below 88: the reference's loss exponentiates them without subtracting the
    # row maximum (ewops.h:243) and returns NaN beyond that, where the kernel under test still gives the loss
    layers, tok, pos = make_model(n_layers, n, ffn, vocab, L, seed=600, tok_std=0.05)
    ids = orc.fill_uniform_int((B, L), 601, 0, vocab - 1)
    labels = orc.fill_uniform_int((B * L,), 602, 0, vocab - 1)
    want_loss, want_logits, want_hidden = orc.model_forward(
        ids, labels, tok, pos, layers, luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"], pre_ln=pre_ln, mask=mask,
        valid_len=valid, operands_bf16=bf16, nthreads=16)
    model = sfb.Model(T(tok), T(pos), [{k: T(v) for k, v in w.items()} for w in layers], luts, bs, H, d, ffn,
                      dtype=sfb.BF16 if bf16 else sfb.F32, max_blocks=4, pre_ln=pre_ln)
    tol = 1e-2 if bf16 else 1e-4
    for _ in range(2):
        out = model.forward(T(ids), T(labels), mask=sfb.to_device(mask), valid_len=sfb.to_device(valid),
                            want_logits=True, want_hidden=True)
        torch.cuda.synchronize()
        assert rel_err(out["hidden"].cpu().numpy(), want_hidden) <= tol
        assert rel_err(out["logits"].cpu().numpy(), want_logits) <= tol
        assert np.isfinite(want_loss) and abs(float(out["loss"]) - want_loss) <= tol * want_loss
    # without labels and without copies: only the workspace is written
    assert model.forward(T(ids)) == {}


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_cpp_whole_model_host_program(dtype):
    """sf-bert_amd/host/transformer_inference: a C++ main in the shape of the reference's
    transformer_inference_part.cpp (same command line) on sfb_model_forward; a freshly initialised model must
    give a loss of ln(256)."""
    import os
    import subprocess
    from sfb import ROOT
    exe = os.path.join(ROOT, "sf-bert_amd", "host", "transformer_inference")
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    out = subprocess.run([exe, "2", "2", "512", "4", "64", dtype], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and "PASSED" in out.stdout
