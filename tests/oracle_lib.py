"""ctypes view of the CPU oracle (oracle/liboracle.so) and, when it was built, of the reference's own
CPU functions (oracle/_ref/libsfbert_ref.so).  Checker only: nothing under sf-bert_amd imports this."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")


def _load():
    path = os.path.join(ORACLE_DIR, "liboracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR], stdout=subprocess.DEVNULL)
    return C.CDLL(path)


lib = _load()
_ref_path = os.path.join(ORACLE_DIR, "_ref", "libsfbert_ref.so")
ref = C.CDLL(_ref_path) if os.path.exists(_ref_path) else None

vp = C.c_void_p
lib.orc_count_blocks.restype = C.c_uint32
lib.orc_build_nn_lut.restype = C.c_uint32
lib.orc_build_tn_lut.restype = C.c_uint32
lib.orc_div64.restype = C.c_uint32
lib.orc_f32_to_bf16_rne.restype = C.c_uint16
lib.orc_f32_to_bf16_rne.argtypes = [C.c_float]
lib.orc_f32_to_bf16_half_away.restype = C.c_uint16
lib.orc_f32_to_bf16_half_away.argtypes = [C.c_float]
lib.orc_bf16_to_f32.restype = C.c_float
lib.orc_bf16_to_f32.argtypes = [C.c_uint16]

MASK_ALL, MASK_CAUSAL_DIAG, MASK_LOCAL, MASK_TRIANGULAR_ALL = 0, 1, 2, 3


def _p(a):
    return None if a is None else a.ctypes.data_as(vp)


# ---------------------------------------------------------------- layouts
def layout_full(nb, causal=True):
    out = np.zeros((nb, nb), np.uint32)
    lib.orc_layout_full(_p(out), nb, int(causal))
    return out


def layout_local(nb, extra_diag, bidirectional=False):
    out = np.zeros((nb, nb), np.uint32)
    lib.orc_layout_local(_p(out), nb, extra_diag, int(bidirectional))
    return out


def layout_fixed(heads, nb, stride, causal=True):
    out = np.zeros((heads, nb, nb), np.uint32)
    lib.orc_layout_fixed(_p(out), heads, nb, stride, int(causal))
    return out


def layout_strided_chunks(nb, block_chunks):
    out = np.zeros((nb, nb), np.uint32)
    lib.orc_layout_strided_chunks(_p(out), nb, block_chunks)
    return out


def layout_strided(nb, band, stride, causal=False):
    out = np.zeros((nb, nb), np.uint32)
    lib.orc_layout_strided(_p(out), nb, band, stride, int(causal))
    return out


def bigbird_draw(nb, window, nglobal, both_ends, nrand, seed):
    out = np.zeros((nb, max(nrand, 1)), np.int32)
    lib.orc_bigbird_draw(_p(out), nb, window, nglobal, int(both_ends), nrand, C.c_uint64(seed))
    return out[:, :nrand]


def layout_bigbird(nb, window, nglobal, both_ends, rand_cols=None):
    out = np.zeros((nb, nb), np.uint32)
    nrand = 0 if rand_cols is None else rand_cols.shape[1]
    rc = None if rand_cols is None else np.ascontiguousarray(rand_cols, np.int32)
    lib.orc_layout_bigbird(_p(out), nb, window, nglobal, int(both_ends), _p(rc), nrand)
    return out


# ---------------------------------------------------------------- LUTs / masks
def build_luts(layout, nn_max_init=0):
    """layout [nb,nb] -> dict(nt_lut [blocks,2], nn_lut [nb+blocks,2], nn_max, rblk_lut, blocks)."""
    layout = np.ascontiguousarray(layout, np.uint32)
    nb = layout.shape[0]
    blocks = int(lib.orc_count_blocks(_p(layout), nb))
    nt = np.zeros((max(blocks, 1), 2), np.uint32)
    lib.orc_build_nt_lut(_p(nt), _p(layout), nb)
    nt = nt[:blocks]
    nn = np.zeros((nb + blocks, 2), np.uint32)
    nn_max = int(lib.orc_build_nn_lut(_p(nn), _p(np.ascontiguousarray(nt)), blocks, nb, nn_max_init))
    rblk = np.zeros((max(blocks, 1), 2), np.uint32)
    lib.orc_build_rblk_lut(_p(rblk), _p(nn), nb)
    return dict(nt_lut=nt, nn_lut=nn, nn_max=nn_max, rblk_lut=rblk[:blocks], blocks=blocks, nb=nb)


def element_mask(nt_lut, bs, kind, local_attn_ctx=0):
    blocks = nt_lut.shape[0]
    keep = np.zeros((blocks, bs, bs), np.uint8)
    lib.orc_element_mask(_p(keep), _p(np.ascontiguousarray(nt_lut)), blocks, bs, kind, local_attn_ctx)
    return keep


def pack_mask(keep):
    blocks, bs, _ = keep.shape
    wb = max(bs // 8, 1)
    words = np.zeros(blocks * bs, {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[wb])
    lib.orc_pack_mask(_p(words), _p(np.ascontiguousarray(keep)), blocks, bs, wb)
    return words


def transpose_mask(words, blocks, bs):
    out = np.zeros_like(words)
    lib.orc_transpose_mask(_p(out), _p(words), blocks, bs, words.dtype.itemsize)
    return out


def magicu64(d):
    m, s = C.c_uint32(0), C.c_uint32(0)
    lib.orc_magicu64(d, C.byref(m), C.byref(s))
    return m.value, s.value


# ---------------------------------------------------------------- attention
def attention(Q, K, V, nn_lut, bs, scale, mask=None, valid_len=None, lut_heads=1, mask_heads=1,
              blocks=None, nthreads=1):
    B, L, H, d = Q.shape
    nb = L // bs
    nn_lut = np.ascontiguousarray(nn_lut, np.uint32)
    if blocks is None:
        blocks = nn_lut.reshape(-1, 2).shape[0] // lut_heads - nb
    O = np.zeros_like(Q)
    wb = 0 if mask is None else mask.dtype.itemsize
    vl = None if valid_len is None else np.ascontiguousarray(valid_len, np.int32)
    lib.orc_blocksparse_attention(_p(O), _p(Q), _p(K), _p(V), _p(nn_lut), _p(mask), wb, _p(vl), B, L,
                                  H, d, bs, C.c_float(scale), lut_heads, blocks + nb, mask_heads,
                                  blocks, nthreads)
    return O


def sdd_nt(Q, K, nt_lut, bs, lut_heads=1):
    B, L, H, d = Q.shape
    nt_lut = np.ascontiguousarray(nt_lut, np.uint32)
    blocks = nt_lut.reshape(-1, 2).shape[0] // lut_heads
    S = np.zeros((B, H, blocks, bs, bs), np.float32)
    lib.orc_sdd_nt(_p(S), _p(Q), _p(K), _p(nt_lut), B, L, H, d, bs, blocks, lut_heads)
    return S


def masked_softmax(S, nn_lut, nb, scale, mask=None, valid_len=None, lut_heads=1, mask_heads=1):
    B, H, blocks, bs, _ = S.shape
    P = np.zeros_like(S)
    wb = 0 if mask is None else mask.dtype.itemsize
    vl = None if valid_len is None else np.ascontiguousarray(valid_len, np.int32)
    lib.orc_masked_softmax(_p(P), _p(S), _p(np.ascontiguousarray(nn_lut, np.uint32)), _p(mask), wb,
                           _p(vl), B, H, nb, bs, blocks, C.c_float(scale), lut_heads, mask_heads)
    return P


def dsd_nn(P, V, nn_lut, lut_heads=1):
    B, H, blocks, bs, _ = P.shape
    _, L, _, d = V.shape
    O = np.zeros_like(V)
    lib.orc_dsd_nn(_p(O), _p(P), _p(V), _p(np.ascontiguousarray(nn_lut, np.uint32)), B, L, H, d, bs,
                   blocks, lut_heads)
    return O


# ---------------------------------------------------------------- layer ops
def build_tn_lut(nt_lut, nb):
    nt_lut = np.ascontiguousarray(nt_lut, np.uint32)
    blocks = nt_lut.shape[0]
    tn = np.zeros((nb + blocks, 2), np.uint32)
    tn_max = lib.orc_build_tn_lut(_p(tn), _p(nt_lut), blocks, nb)
    return tn, int(tn_max)


def masked_softmax_grad(dP, P, nn_lut, nb, scale, lut_heads=1):
    B, H, blocks, bs, _ = P.shape
    dS = np.zeros_like(P)
    lib.orc_masked_softmax_grad(_p(dS), _p(np.ascontiguousarray(dP, np.float32)), _p(P),
                                _p(np.ascontiguousarray(nn_lut, np.uint32)), B, H, nb, bs, blocks,
                                C.c_float(scale), lut_heads)
    return dS


def dsd_tn(A, X, tn_lut, lut_heads=1):
    B, H, blocks, bs, _ = A.shape
    _, L, _, d = X.shape
    out = np.zeros((B, L, H, d), np.float32)
    lib.orc_dsd_tn(_p(out), _p(A), _p(X), _p(np.ascontiguousarray(tn_lut, np.uint32)), B, L, H, d, bs,
                   blocks, lut_heads)
    return out


def attention_backward(Q, K, V, dO, luts, bs, scale, mask=None, valid_len=None):
    """Gradients of the unfused path in the reference's order (transformer_attention_optimize.cu:924-964):
    dV = P^T dO, dP = dO V^T, dS = softmax_grad(dP, P), dK = dS^T Q, dQ = dS K.  Returns dQ, dK, dV, P."""
    nb = Q.shape[1] // bs
    S = sdd_nt(Q, K, luts["nt_lut"], bs)
    P = masked_softmax(S, luts["nn_lut"], nb, scale, mask=mask, valid_len=valid_len)
    tn, _ = build_tn_lut(luts["nt_lut"], nb)
    dV = dsd_tn(P, dO, tn)
    dP = sdd_nt(dO, V, luts["nt_lut"], bs)
    dS = masked_softmax_grad(dP, P, luts["nn_lut"], nb, scale)
    dK = dsd_tn(dS, Q, tn)
    dQ = dsd_nn(dS, K, luts["nn_lut"])
    return dQ, dK, dV, P


def layernorm(x, g, b):
    rows, state = x.reshape(-1, x.shape[-1]).shape
    out = np.zeros_like(x)
    mean = np.zeros(rows, np.float32)
    rstd = np.zeros(rows, np.float32)
    lib.orc_layernorm(_p(out), _p(mean), _p(rstd), _p(x), _p(g), _p(b), rows, state)
    return out, mean, rstd


def gelu(x):
    out = np.zeros_like(x)
    lib.orc_gelu(_p(out), _p(x), C.c_long(x.size))
    return out


def bias(x, b):
    out = np.zeros_like(x)
    lib.orc_bias(_p(out), _p(x), _p(b), x.shape[-1], x.size // x.shape[-1])
    return out


def sgemm(A, W, nthreads=1):
    m, k = A.shape
    n = W.shape[1]
    out = np.zeros((m, n), np.float32)
    lib.orc_sgemm(_p(out), _p(A), _p(W), m, n, k, nthreads)
    return out


def round_bf16(x):
    y = np.ascontiguousarray(x, np.float32).copy()
    lib.orc_round_to_bf16_rne(_p(y), C.c_long(y.size))
    return y


class LayerWeights(C.Structure):
    _fields_ = [(n, vp) for n in ("wq", "wk", "wv", "wo", "w1", "w2", "bq", "bk", "bv", "bo", "b1",
                                  "b2", "ln1_g", "ln1_b", "ln2_g", "ln2_b")]


def encoder_layer(x, weights, nn_lut, B, L, H, d, ffn, bs, blocks, mask=None, valid_len=None,
                  operands_bf16=False, nthreads=1):
    keep = [np.ascontiguousarray(v, np.float32) for v in weights.values()]
    w = LayerWeights(**{k: _p(a) for k, a in zip(weights.keys(), keep)})
    y = np.zeros_like(x)
    wb = 0 if mask is None else mask.dtype.itemsize
    vl = None if valid_len is None else np.ascontiguousarray(valid_len, np.int32)
    lib.orc_encoder_layer(_p(y), _p(x), C.byref(w), _p(np.ascontiguousarray(nn_lut, np.uint32)),
                          _p(mask), wb, _p(vl), B, L, H, d, ffn, bs, blocks, int(operands_bf16),
                          nthreads)
    return y


def encoder_layer_pre_ln(x, weights, nn_lut, B, L, H, d, ffn, bs, blocks, mask=None, valid_len=None,
                         operands_bf16=False, nthreads=1):
    keep = [np.ascontiguousarray(v, np.float32) for v in weights.values()]
    w = LayerWeights(**{k: _p(a) for k, a in zip(weights.keys(), keep)})
    y = np.zeros_like(x)
    wb = 0 if mask is None else mask.dtype.itemsize
    vl = None if valid_len is None else np.ascontiguousarray(valid_len, np.int32)
    lib.orc_encoder_layer_pre_ln(_p(y), _p(x), C.byref(w), _p(np.ascontiguousarray(nn_lut, np.uint32)),
                                 _p(mask), wb, _p(vl), B, L, H, d, ffn, bs, blocks, int(operands_bf16), nthreads)
    return y


def sgemm_nt(A, W, nthreads=1):
    m, k = A.shape
    n = W.shape[0]
    out = np.zeros((m, n), np.float32)
    lib.orc_sgemm_nt(_p(out), _p(A), _p(W), m, n, k, nthreads)
    return out


def softmax_cross_entropy(logits, labels, want_grad=False):
    """(mean loss, row losses[, softmax - onehot]) of ewops.h:233-261."""
    rows, vocab = logits.shape
    row_loss = np.zeros(rows, np.float32)
    d = np.zeros_like(logits) if want_grad else None
    lib.orc_softmax_cross_entropy.restype = C.c_float
    loss = lib.orc_softmax_cross_entropy(_p(d), _p(row_loss), _p(np.ascontiguousarray(logits, np.float32)),
                                         _p(np.ascontiguousarray(labels, np.int32)), C.c_long(rows), vocab)
    return (np.float32(loss), row_loss, d) if want_grad else (np.float32(loss), row_loss)


def model_forward(ids, labels, tok, pos, layers, nn_lut, B, L, H, d, ffn, bs, blocks, pre_ln=True, mask=None,
                  valid_len=None, operands_bf16=False, nthreads=1):
    """(loss, logits [tokens, vocab], hidden [tokens, state]); layers: list of weight dicts."""
    n, vocab = H * d, tok.shape[0]
    keep = [[np.ascontiguousarray(v, np.float32) for v in w.values()] for w in layers]
    arr = (LayerWeights * len(layers))(*[LayerWeights(**{k: _p(a) for k, a in zip(w.keys(), kp)})
                                         for w, kp in zip(layers, keep)])
    logits = np.zeros((B * L, vocab), np.float32)
    hidden = np.zeros((B * L, n), np.float32)
    wb = 0 if mask is None else mask.dtype.itemsize
    vl = None if valid_len is None else np.ascontiguousarray(valid_len, np.int32)
    lib.orc_model_forward.restype = C.c_float
    loss = lib.orc_model_forward(_p(logits), _p(hidden), _p(np.ascontiguousarray(ids, np.int32)),
                                 _p(np.ascontiguousarray(labels, np.int32)), _p(np.ascontiguousarray(tok, np.float32)),
                                 _p(np.ascontiguousarray(pos, np.float32)), arr, len(layers), int(pre_ln),
                                 _p(np.ascontiguousarray(nn_lut, np.uint32)), _p(mask), wb, _p(vl), B, L, H, d, ffn,
                                 bs, blocks, vocab, int(operands_bf16), nthreads)
    return np.float32(loss), logits, hidden


def fill_normal(shape, seed, std=1.0):
    x = np.zeros(shape, np.float32)
    lib.orc_fill_normal(_p(x), C.c_long(x.size), C.c_uint64(seed), C.c_float(std))
    return x


def fill_uniform_int(shape, seed, lo, hi):
    x = np.zeros(shape, np.int32)
    lib.orc_fill_uniform_int(_p(x), C.c_long(x.size), C.c_uint64(seed), lo, hi)
    return x


# ---------------------------------------------------------------- dense brute force (float64)
def dense_keep_matrix(layout, bs, keep_blocks=None, nt_lut=None, valid=None):
    """[L,L] bool: layout bit & element-mask bit & key < valid."""
    nb = layout.shape[0]
    L = nb * bs
    keep = np.kron(layout.astype(bool), np.ones((bs, bs), bool))
    if keep_blocks is not None:
        for blk, (r, c) in enumerate(nt_lut):
            keep[r * bs:(r + 1) * bs, c * bs:(c + 1) * bs] &= keep_blocks[blk].astype(bool)
    if valid is not None:
        keep[:, valid:] = False
    return keep


def dense_attention_f64(Q, K, V, keep_per_batch, scale):
    """float64 restatement of ewops.h:64-98 semantics on a dense masked score matrix."""
    B, L, H, d = Q.shape
    O = np.zeros((B, L, H, d), np.float64)
    for b in range(B):
        keep = keep_per_batch[b] if isinstance(keep_per_batch, (list, tuple)) else keep_per_batch
        for h in range(H):
            q = Q[b, :, h].astype(np.float64)
            k = K[b, :, h].astype(np.float64)
            v = V[b, :, h].astype(np.float64)
            s = q @ k.T
            mx = np.where(keep, s, -1000000.0).max(axis=1, keepdims=True)
            mx = np.maximum(mx, -1000000.0)
            p = np.where(keep, np.exp(np.where(keep, (s - mx) * scale, 0.0)), 0.0)
            p = p / (p.sum(axis=1, keepdims=True) + 1e-6)
            O[b, :, h] = p @ v
    return O
