"""The kernels against the reference's own outputs: the golden fixtures of tests/golden/ were written by the reference's
CPU functions (tests/golden/make_golden.py); here the library -- on the device, or its host build -- is run on the
fixtures' inputs and compared with those outputs directly, without the oracle in between.  `S` is the binding (capi
of the device library or of the host build), `dev` puts a numpy array where that library reads it."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = 1e-4   # fp32 tensors


def rel_err(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def causal_descriptors(S, L, bs):
    """Dense causal attention (transformer.cpp:533-545) as a block layout: the lower block triangle, with the
    element mask of the diagonal blocks."""
    luts = S.build_luts(S.layout_full(L // bs, causal=True))
    return luts, S.pack_mask(S.element_mask(luts["nt_lut"], bs, S.MASK_CAUSAL_DIAG))


FORWARD_FIXTURES = ["attention_dense_causal.npz", "attention_dense_causal_block64.npz"]


def attention_forward(S, dev, zeros, fixture=FORWARD_FIXTURES[0]):
    z = np.load(os.path.join(GOLDEN, fixture))
    B, L, H, d = (int(x) for x in z["shape"])
    bs, scale = int(z["bs"]), float(z["scale"])
    luts, mask = causal_descriptors(S, L, bs)
    nb, blocks = L // bs, luts["blocks"]
    q, k, v = dev(z["Q"]), dev(z["K"]), dev(z["V"])
    nn, nt, m = S.to_device(luts["nn_lut"]), S.to_device(luts["nt_lut"]), S.to_device(mask)
    want = z["O"]
    assert rel_err(S.fused_attention(q, k, v, nn, bs, blocks, scale, mask=m).cpu().numpy(), want) <= TOL
    sched = S.build_schedule(luts["nn_lut"], nb, 2)
    ws = zeros(S.schedule_workspace_bytes(sched, B, H, bs, d))
    got = S.fused_attention_scheduled(q, k, v, nn, S.to_device(sched["items"]), sched, ws, bs, blocks, scale, mask=m)
    assert rel_err(got.cpu().numpy(), want) <= TOL
    stream = S.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=8, d=d, bf16=False, masked=True)
    sw = zeros(S.stream_workspace_bytes(stream, d))
    got = S.fused_attention_streamed(q, k, v, nn, S.to_device(stream["blob"]), stream, sw, bs, blocks, scale, mask=m)
    assert S.stream_status(stream, d, sw) == 0 and rel_err(got.cpu().numpy(), want) <= TOL
    # the unfused sequence: the softmax takes the mask row-major (blocksparse.h:459-722)
    scores = S.bst_sgemm_nt(nt, q, k, bs, blocks)
    p = S.BlocksparseMaskedSoftmax(nn, S.to_device(S.transpose_mask(mask, blocks, bs)), scores, nb, scale)
    assert rel_err(S.bst_sgemm_xn(nn, p, v, nb).cpu().numpy(), want) <= TOL
    # the same product over work items, block-rows of more than 2 blocks cut
    got = S.bst_sgemm_xn_scheduled(nn, p, v, nb, S.to_device(sched["items"]), sched,
                                   zeros(S.dsd_workspace_bytes(sched, B, H, bs, d)))
    assert rel_err(got.cpu().numpy(), want) <= TOL
    p2 = S.fusion_attention2(nn, q, k, bs, blocks, scale, mask=m)
    assert rel_err(S.bst_sgemm_xn(nn, p2, v, nb).cpu().numpy(), want) <= TOL


def attention_backward(S, dev, zeros, fixture=FORWARD_FIXTURES[0]):
    z = np.load(os.path.join(GOLDEN, fixture))
    g = z if "dQ" in z.files else np.load(os.path.join(GOLDEN, "attention_backward_dense_causal.npz"))
    B, L, H, d = (int(x) for x in z["shape"])
    bs, scale = int(z["bs"]), float(z["scale"])
    luts, mask = causal_descriptors(S, L, bs)
    nb, blocks = L // bs, luts["blocks"]
    q, k, v, do = dev(z["Q"]), dev(z["K"]), dev(z["V"]), dev(g["dO"])
    ld = {name: S.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    m = S.to_device(mask)
    # fused: forward with its log-sum-exp, then dQ, dK, dV in one pass (whole lines, and lines cut in chunks of 2)
    sched = S.build_schedule(luts["nn_lut"], nb, 2)
    ws = zeros(S.schedule_workspace_bytes(sched, B, H, bs, d))
    o, lse = S.fused_attention_forward_lse(q, k, v, ld["nn_lut"], S.to_device(sched["items"]), sched, ws, bs, blocks, scale,
                                           mask=m)
    for cut in (False, True):
        rs = cs = None
        if cut:
            rs, cs = S.build_schedule(luts["nn_lut"], nb, 2), S.build_schedule(luts["tn_lut"], nb, 2)
            rs["items_dev"], cs["items_dev"] = S.to_device(rs["items"]), S.to_device(cs["items"])
        dq, dk, dv = S.fused_attention_backward(q, k, v, o, do, lse, ld["nn_lut"], ld["tn_lut"], bs, blocks, scale, mask=m,
                                                row_sched=rs, col_sched=cs)
        for name, got in (("dQ", dq), ("dK", dk), ("dV", dv)):
            assert rel_err(got.cpu().numpy(), g[name]) <= TOL, (name, cut)
    # the reference's sequence (transformer_attention_optimize.cu:924-965) from the stored probabilities
    p = S.fusion_attention2(ld["nn_lut"], q, k, bs, blocks, scale, mask=m)
    dq, dk, dv = S.attention_backward(q, k, v, do, p, ld, bs, blocks, scale)
    for name, got in (("dQ", dq), ("dK", dk), ("dV", dv)):
        assert rel_err(got.cpu().numpy(), g[name]) <= TOL, name


def layer_ops(S, dev):
    z = np.load(os.path.join(GOLDEN, "layer_ops.npz"))
    x, gain, beta = dev(z["x"]), dev(z["g"]), dev(z["b"])
    out, mean, rstd = S.layernorm(x, gain, beta, return_stats=True)
    assert rel_err(out.cpu().numpy(), z["layernorm"]) <= 1e-5
    assert rel_err(mean.cpu().numpy(), z["mean"]) <= 1e-5 and rel_err(rstd.cpu().numpy(), z["rstd"]) <= 1e-5
    assert rel_err(S.gelu(x).cpu().numpy(), z["gelu"]) <= 1e-5
    assert rel_err(S.bias(x, gain).cpu().numpy(), z["bias"]) <= 1e-6


def cross_entropy(S, dev):
    z = np.load(os.path.join(GOLDEN, "softmax_cross_entropy.npz"))
    loss, _, grad = S.softmax_cross_entropy(dev(z["logits"]), dev(z["labels"]), want_grad=True)
    assert abs(float(loss) - float(z["loss"])) <= 1e-5 * float(z["loss"])
    assert rel_err(grad.cpu().numpy(), z["grad"]) <= 1e-5
