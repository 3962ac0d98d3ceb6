"""Encoder-layer ops, the GEMM seam and the whole layer against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, rel_err
from sfb import sfb

pytestmark = pytest.mark.gpu
T = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_layer_ops_match_oracle():
    rows, state = 515, 768
    x = orc.fill_normal((rows, state), 1) * 2 + 0.3
    g = orc.fill_normal((state,), 2) + 1
    b = orc.fill_normal((state,), 3)
    want, mean, rstd = orc.layernorm(x, g, b)
    got, m2, r2 = sfb.layernorm(T(x), T(g), T(b), return_stats=True)
    assert rel_err(got.cpu().numpy(), want) <= 1e-5
    assert rel_err(m2.cpu().numpy(), mean) <= 1e-5 and rel_err(r2.cpu().numpy(), rstd) <= 1e-5
    assert rel_err(sfb.gelu(T(x)).cpu().numpy(), orc.gelu(x)) <= 1e-6
    assert np.array_equal(sfb.bias(T(x), T(b)).cpu().numpy(), orc.bias(x, b))
    y = orc.fill_normal((rows, state), 4)
    assert np.array_equal(sfb.tensor_add_tensor(T(x), T(y)).cpu().numpy(), x + y)
    fused = sfb.bias_act(T(x), bias=T(b), residual=T(y), act=1).cpu().numpy()
    assert rel_err(fused, orc.gelu(orc.bias(x, b)) + y) <= 1e-6
    as_bf16 = sfb.bias_act(T(x), bias=T(b), out_dtype=sfb.BF16).float().cpu().numpy()
    assert np.array_equal(as_bf16, orc.round_bf16(orc.bias(x, b)))
    assert np.array_equal(sfb.cast_bf16(T(x)).float().cpu().numpy(), orc.round_bf16(x))
    ln_bf16 = sfb.layernorm(T(x), T(g), T(b), out_dtype=sfb.BF16).float().cpu().numpy()
    assert rel_err(ln_bf16, want) <= 4e-3


@pytest.mark.parametrize("state", [64, 768, 1024, 2048])
def test_bias_residual_layernorm_one_pass(state):
    """The fused kernel equals bias -> tensor_add_tensor -> layernorm of the oracle, and bit for bit the
    two-kernel sequence of the library; its bf16 copy is the fp32 result rounded to nearest even."""
    rows = 131
    x = orc.fill_normal((rows, state), 11) * 1.5
    res = orc.fill_normal((rows, state), 12) + 0.2
    bias = orc.fill_normal((state,), 13)
    g = orc.fill_normal((state,), 14) + 1
    b = orc.fill_normal((state,), 15)
    want, _, _ = orc.layernorm(orc.bias(x, bias) + res, g, b)
    got, got16 = sfb.bias_residual_layernorm(T(x), T(bias), T(res), T(g), T(b), with_bf16=True)
    assert rel_err(got.cpu().numpy(), want) <= 1e-5
    two = sfb.layernorm(sfb.bias_act(T(x), bias=T(bias), residual=T(res)), T(g), T(b))
    assert np.array_equal(got.cpu().numpy(), two.cpu().numpy())
    assert np.array_equal(got16.float().cpu().numpy(), orc.round_bf16(got.cpu().numpy()))
    plain = sfb.bias_residual_layernorm(T(x), None, None, T(g), T(b))
    assert rel_err(plain.cpu().numpy(), orc.layernorm(x, g, b)[0]) <= 1e-5
    with pytest.raises(sfb.SfbError):
        sfb.bias_residual_layernorm(T(orc.fill_normal((4, 4096), 1)), None, None, T(orc.fill_normal((4096,), 2)),
                                    T(orc.fill_normal((4096,), 3)))


def test_embedding_and_position_add():
    vocab, state, B, L = 1000, 768, 3, 64
    table = orc.fill_normal((vocab, state), 5)
    pos = orc.fill_normal((L, state), 6)
    ids = orc.fill_uniform_int((B, L), 7, 0, vocab - 1)
    got = sfb.embedding_lookup(T(table), T(ids), T(pos)).cpu().numpy()
    assert np.array_equal(got, table[ids] + pos[None])
    assert np.array_equal(sfb.embedding_lookup(T(table), T(ids)).cpu().numpy(), table[ids])
    x = orc.fill_normal((B, L, state), 8)
    assert np.array_equal(sfb.tensor_add_matrix(T(x), T(pos)).cpu().numpy(), x + pos[None])


def test_transpose_0123to0213():
    # bit-exact copy; checked against the oracle (itself pinned to the reference's loop) and against numpy
    for shape in ((2, 5, 3, 4), (2, 128, 12, 64), (1, 12, 96, 32)):
        src = orc.fill_normal(shape, 31)
        want = np.zeros((shape[0], shape[2], shape[1], shape[3]), np.float32)
        orc.lib.orc_transpose_0213(orc._p(src), orc._p(want), *shape)
        got = sfb.transpose_0123to0213(T(src)).cpu().numpy()
        assert np.array_equal(got, want) and np.array_equal(got, src.transpose(0, 2, 1, 3))
        # applying it twice with the middle sizes swapped restores the input
        back = sfb.transpose_0123to0213(sfb.transpose_0123to0213(T(src))).cpu().numpy()
        assert np.array_equal(back, src)
    with pytest.raises(sfb.SfbError):
        sfb.transpose_0123to0213(T(np.zeros((2, 3, 4, 6), np.float32)))   # last size not a multiple of 4


@pytest.mark.parametrize("bf16", [False, True])
def test_gemm_matches_oracle(bf16):
    m, k, n = 200, 768, 3072
    A = orc.fill_normal((m, k), 9)
    W = orc.fill_normal((k, n), 10, 0.02)
    if bf16:
        A, W = orc.round_bf16(A), orc.round_bf16(W)
    want = orc.sgemm(A, W, nthreads=16)
    a, w = T(A), T(W)
    if bf16:
        a, w = a.to(torch.bfloat16), w.to(torch.bfloat16)
    got = sfb.gemm(a, w).cpu().numpy()
    assert rel_err(got, want) <= 1e-5
    want64 = A.astype(np.float64) @ W.astype(np.float64)
    assert rel_err(got, want64) <= 1e-5


@pytest.mark.parametrize("bf16,out_bf16", [(False, False), (True, True), (True, False)])
def test_gemm_bias_one_kernel(bf16, out_bf16):
    """GEMM with bias (and rounding to bf16) in the epilogue equals sgemm -> bias (-> one rounding) of the oracle."""
    m, k, n = 520, 768, 768
    A = orc.fill_normal((m, k), 19)
    W = orc.fill_normal((k, n), 20, 0.02)
    b = orc.fill_normal((n,), 21)
    if bf16:
        A, W = orc.round_bf16(A), orc.round_bf16(W)
    want = orc.bias(orc.sgemm(A, W, nthreads=16), b)
    a, w = T(A), T(W)
    if bf16:
        a, w = a.to(torch.bfloat16), w.to(torch.bfloat16)
    got = sfb.gemm_bias(a, w, T(b), out_dtype=sfb.BF16 if out_bf16 else sfb.F32)
    assert got.dtype == (torch.bfloat16 if out_bf16 else torch.float32)
    got = got.float().cpu().numpy()
    if out_bf16:
        # one rounding of the fp32 result: at most one bf16 step away from the rounded oracle value
        assert np.abs(got - orc.round_bf16(want)).max() <= 2.0 ** -8 * np.abs(want).max()
        assert np.array_equal(got, orc.round_bf16(got))
    else:
        assert rel_err(got, want) <= 1e-5


@pytest.mark.parametrize("bf16,out_bf16", [(False, False), (True, False), (True, True)])
def test_gemm_bias_gelu_one_kernel(bf16, out_bf16):
    """GEMM with bias and the sigmoid-form GELU in the epilogue equals sgemm -> bias -> gelu of the oracle (values
    chosen so that the activation's curved part, |x| < 1, and both tails are covered)."""
    m, k, n = 520, 768, 3072
    A = orc.fill_normal((m, k), 23)
    W = orc.fill_normal((k, n), 24, 0.08)
    b = orc.fill_normal((n,), 25)
    if bf16:
        A, W = orc.round_bf16(A), orc.round_bf16(W)
    pre = orc.bias(orc.sgemm(A, W, nthreads=16), b)
    assert (np.abs(pre) < 1).mean() > 0.2 and (pre > 3).mean() > 0.01 and (pre < -3).mean() > 0.01
    want = orc.gelu(pre)
    a, w = T(A), T(W)
    if bf16:
        a, w = a.to(torch.bfloat16), w.to(torch.bfloat16)
    code = sfb.BF16 if out_bf16 else sfb.F32

    def check(got, scale):
        assert got.dtype == (torch.bfloat16 if out_bf16 else torch.float32)
        got = got.float().cpu().numpy()
        if out_bf16:
            assert np.array_equal(got, orc.round_bf16(got))
            assert np.abs(got / scale - want).max() <= 2.0 ** -8 * np.abs(want).max()
        else:
            assert rel_err(got / scale, want) <= 1e-5

    # the scaled form runs wherever the GEMM library has a Swish epilogue; its factor is 1 or the slope
    got, scale = sfb.gemm_bias_gelu_scaled(a, w, T(b), out_dtype=code)
    assert scale in (1.0, np.float32(1.702))
    check(got, np.float32(scale))
    # the exact form needs the library's slope argument for bf16 output and says so when it is missing
    try:
        check(sfb.gemm_bias_gelu(a, w, T(b), out_dtype=code), np.float32(1.0))
    except sfb.SfbError as e:
        assert out_bf16 and scale != 1.0 and e.status == 7, e


def layer_weights(n, ffn, seed):
    shapes = [("wq", (n, n)), ("wk", (n, n)), ("wv", (n, n)), ("wo", (n, n)), ("w1", (n, ffn)), ("w2", (ffn, n)),
              ("bq", (n,)), ("bk", (n,)), ("bv", (n,)), ("bo", (n,)), ("b1", (ffn,)), ("b2", (n,)),
              ("ln1_g", (n,)), ("ln1_b", (n,)), ("ln2_g", (n,)), ("ln2_b", (n,))]
    w = {k: orc.fill_normal(s, seed + i, 0.02) for i, (k, s) in enumerate(shapes)}
    w["ln1_g"] = w["ln1_g"] + 1
    w["ln2_g"] = w["ln2_g"] + 1
    return w


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("max_blocks", [0, 4])
def test_encoder_layer_matches_oracle(bf16, max_blocks):
    # BERT-base widths (hidden 768, 12 heads, d 64, FFN 3072), BigBird attention, short sequence
    B, L, H, d, ffn, bs = 2, 1024, 12, 64, 3072, 64
    n, nb = H * d, L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    w = layer_weights(n, ffn, 100)
    x = orc.fill_normal((B * L, n), 300)
    want = orc.encoder_layer(x, w, luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"], operands_bf16=bf16,
                             nthreads=16)
    layer = sfb.EncoderLayer({k: T(v) for k, v in w.items()}, luts, bs, H, d, ffn,
                             dtype=sfb.BF16 if bf16 else sfb.F32, max_blocks=max_blocks)
    for _ in range(2):
        got = layer.forward(T(x), B, L).cpu().numpy()
        torch.cuda.synchronize()
        err = rel_err(got, want)
        print("layer rel err", err)
        assert err <= (1e-2 if bf16 else 1e-4)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("pre_ln", [False, True])
def test_encoder_layer_streamed_matches_oracle(bf16, pre_ln):
    """The layer with its attention launched over streams (sfb_encoder_layer_forward_streamed), both wirings."""
    B, L, H, d, ffn, bs = 2, 1024, 12, 64, 3072, 64
    n, nb = H * d, L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    w = layer_weights(n, ffn, 100)
    x = orc.fill_normal((B * L, n), 300)
    oracle = orc.encoder_layer_pre_ln if pre_ln else orc.encoder_layer
    want = oracle(x, w, luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"], operands_bf16=bf16, nthreads=16)
    layer = sfb.EncoderLayer({k: T(v) for k, v in w.items()}, luts, bs, H, d, ffn,
                             dtype=sfb.BF16 if bf16 else sfb.F32, pre_ln=pre_ln, streamed=True)
    for _ in range(2):
        got = layer.forward(T(x), B, L).cpu().numpy()
        torch.cuda.synchronize()
        assert rel_err(got, want) <= (1e-2 if bf16 else 1e-4)


@pytest.mark.parametrize("pre_ln", [False, True])
@pytest.mark.parametrize("bf16", [False, True])
def test_encoder_layer_merged_qkv_product(bf16, pre_ln):
    """Q, K and V as one product (sfb_pack_qkv, the attention reading column slices of its result): same result as
    the three products of transformer.cpp:516-522, both wirings, and the oracle's within tolerance."""
    B, L, H, d, ffn, bs = 2, 1024, 12, 64, 3072, 64
    n, nb = H * d, L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    w = layer_weights(n, ffn, 120)
    for name in ("bq", "bk", "bv"):
        w[name] = orc.fill_normal((n,), 121 + len(name) + ord(name[1])) * 0.1   # distinct biases: a mix-up shows
    x = orc.fill_normal((B * L, n), 320)
    oracle = orc.encoder_layer_pre_ln if pre_ln else orc.encoder_layer
    want = oracle(x, w, luts["nn_lut"], B, L, H, d, ffn, bs, luts["blocks"], operands_bf16=bf16, nthreads=16)
    outs = []
    for merge in (False, True):
        layer = sfb.EncoderLayer({k: T(v) for k, v in w.items()}, luts, bs, H, d, ffn,
                                 dtype=sfb.BF16 if bf16 else sfb.F32, pre_ln=pre_ln, max_blocks=4, merge_qkv=merge)
        assert (layer.c_weights.wqkv is not None) == merge
        outs.append(layer.forward(T(x), B, L))
        torch.cuda.synchronize()
        assert rel_err(outs[-1].cpu().numpy(), want) <= (1e-2 if bf16 else 1e-4)
    # the same products over the same k, only laid side by side: bf16 identical, fp32 to rounding of another kernel
    assert float((outs[0] - outs[1]).abs().max()) <= (0 if bf16 else 1e-4) * float(outs[0].abs().max())


def test_encoder_layer_per_head_luts_and_masks():
    """The reference's `fixed` pattern gives every head its own layout and mask (fixed_fusion_test.cu:38-39, 58-106):
    the streamed layer against the same layer put together from the oracle's operations (fp32)."""
    B, L, H, d, ffn, bs = 2, 512, 4, 64, 512, 32
    n, nb = H * d, L // bs
    lay = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lay[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    nn = np.concatenate([p["nn_lut"] for p in per_head])
    masks = np.concatenate([sfb.pack_mask(sfb.element_mask(p["nt_lut"], bs, sfb.MASK_CAUSAL_DIAG)) for p in per_head])
    w = layer_weights(n, ffn, 500)
    x = orc.fill_normal((B * L, n), 700)

    def proj(a, wn, bn):
        return orc.bias(orc.sgemm(a, w[wn], nthreads=16), w[bn])
    q, k, v = (proj(x, "w" + c, "b" + c).reshape(B, L, H, d) for c in "qkv")
    attn = orc.attention(q, k, v, nn, bs, 1.0 / np.sqrt(d), mask=masks, lut_heads=H, mask_heads=H, blocks=blocks,
                         nthreads=16).reshape(B * L, n)
    x1 = orc.layernorm(x + proj(attn, "wo", "bo"), w["ln1_g"], w["ln1_b"])[0]
    want = orc.layernorm(x1 + proj(orc.gelu(proj(x1, "w1", "b1")), "w2", "b2"), w["ln2_g"], w["ln2_b"])[0]

    luts = sfb.Luts(nn_lut=nn, blocks=blocks, nb=nb)
    layer = sfb.EncoderLayer({k_: T(v_) for k_, v_ in w.items()}, luts, bs, H, d, ffn, dtype=sfb.F32, streamed=True,
                             lut_heads=H, mask_heads=H)
    got = layer.forward(T(x), B, L, mask=sfb.to_device(masks)).cpu().numpy()
    torch.cuda.synchronize()
    assert rel_err(got, want) <= 1e-4
    # the same in bf16 against the fp32 result (operand rounding only)
    layer16 = sfb.EncoderLayer({k_: T(v_) for k_, v_ in w.items()}, luts, bs, H, d, ffn, dtype=sfb.BF16, streamed=True,
                               lut_heads=H, mask_heads=H)
    got16 = layer16.forward(T(x), B, L, mask=sfb.to_device(masks)).cpu().numpy()
    torch.cuda.synchronize()
    assert rel_err(got16, want) <= 2e-2
