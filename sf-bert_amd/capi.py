"""ctypes binding of libsfbert_hip.so and a thin host mirror of the reference's operator surface.

Descriptor builders work on numpy arrays (host integer code).  Device entry points take torch CUDA
tensors purely as device memory; the launch goes on torch's current stream.  Function and argument
names follow the reference launchers (bst_sgemm_nt, BlocksparseMaskedSoftmax, bst_sgemm_xn,
fusion_attention*: openai_blocksparse.h:202, blocksparse.h:649,965, fusion_blocksparse.h:400-3050).
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# SFBERT_HIP_LIB points at an alternative build of the same library (e.g. an experimental kernel variant)
LIB_PATH = os.environ.get("SFBERT_HIP_LIB") or os.path.join(_HERE, "libsfbert_hip.so")

F32, BF16 = 0, 1
NT_OP, NN_OP, TN_OP = 0, 1, 2
MASK_ALL, MASK_CAUSAL_DIAG, MASK_LOCAL, MASK_TRIANGULAR_ALL = 0, 1, 2, 3


class SfbError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = lib.sfb_status_string(status).decode() if lib is not None else "?"
        super().__init__("%s failed: status %d (%s)" % (where, status, msg))


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libsfbert_hip.so is not built (%s); run `python __graft_entry__.py` or "
            "`python sf-bert_amd/build.py`. There is no fallback path." % LIB_PATH)
    return C.CDLL(LIB_PATH)


lib = _load()
lib.sfb_status_string.restype = C.c_char_p
lib.sfb_status_string.argtypes = [C.c_int]
lib.sfb_count_blocks.restype = C.c_uint32
lib.sfb_magicu64.restype = None
lib.sfb_schedule_workspace_bytes.restype = C.c_size_t

#: every symbol include/sfbert_hip.h declares (checked by the CPU test-suite)
EXPORTED = [
    "sfb_status_string", "sfb_device_available",
    "sfb_layout_full", "sfb_layout_local", "sfb_layout_fixed", "sfb_layout_strided_chunks",
    "sfb_layout_strided", "sfb_layout_bigbird", "sfb_bigbird_draw", "sfb_count_blocks",
    "sfb_build_nt_lut", "sfb_build_nn_lut", "sfb_build_rblk_lut", "sfb_magicu64", "sfb_element_mask",
    "sfb_pack_mask", "sfb_transpose_mask", "sfb_build_row_order",
    "sfb_build_schedule", "sfb_schedule_workspace_bytes",
    "sfb_fused_attention", "sfb_fused_attention_scheduled",
    "sfb_sdd_nt", "sfb_masked_softmax", "sfb_dsd_xn", "sfb_fused_sdd_softmax",
]


def _check(status, where):
    if status != 0:
        raise SfbError(status, where)


def _np(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _dev(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


# ------------------------------------------------------------------------------------ layouts
def layout_full(nb, causal=True):
    out = np.zeros((nb, nb), np.uint32)
    _check(lib.sfb_layout_full(_np(out), nb, int(causal)), "sfb_layout_full")
    return out


def layout_local(nb, extra_diag, bidirectional=False):
    out = np.zeros((nb, nb), np.uint32)
    _check(lib.sfb_layout_local(_np(out), nb, extra_diag, int(bidirectional)), "sfb_layout_local")
    return out


def layout_fixed(heads, nb, stride, causal=True):
    out = np.zeros((heads, nb, nb), np.uint32)
    _check(lib.sfb_layout_fixed(_np(out), heads, nb, stride, int(causal)), "sfb_layout_fixed")
    return out


def layout_strided_chunks(nb, block_chunks):
    out = np.zeros((nb, nb), np.uint32)
    _check(lib.sfb_layout_strided_chunks(_np(out), nb, block_chunks), "sfb_layout_strided_chunks")
    return out


def layout_strided(nb, band, stride, causal=False):
    out = np.zeros((nb, nb), np.uint32)
    _check(lib.sfb_layout_strided(_np(out), nb, band, stride, int(causal)), "sfb_layout_strided")
    return out


def bigbird_draw(nb, window, nglobal, both_ends, nrand, seed):
    out = np.zeros((nb, max(nrand, 1)), np.int32)
    _check(lib.sfb_bigbird_draw(_np(out), nb, window, nglobal, int(both_ends), nrand,
                                C.c_uint64(seed)), "sfb_bigbird_draw")
    return np.ascontiguousarray(out[:, :nrand])


def layout_bigbird(nb, window, nglobal, both_ends, rand_cols=None):
    out = np.zeros((nb, nb), np.uint32)
    nrand = 0 if rand_cols is None else rand_cols.shape[1]
    rc = None if rand_cols is None or nrand == 0 else np.ascontiguousarray(rand_cols, np.int32)
    _check(lib.sfb_layout_bigbird(_np(out), nb, window, nglobal, int(both_ends), _np(rc), nrand),
           "sfb_layout_bigbird")
    return out


# ------------------------------------------------------------------------------------ LUTs / masks
class Luts(dict):
    """nt_lut [blocks,2], nn_lut [nb+blocks,2], rblk_lut [blocks,2], row_order [nb], nn_max, blocks, nb."""
    __getattr__ = dict.__getitem__


def build_luts(layout, nn_max_init=0):
    layout = np.ascontiguousarray(layout, np.uint32)
    nb = layout.shape[0]
    blocks = int(lib.sfb_count_blocks(_np(layout), nb))
    nt = np.zeros((max(blocks, 1), 2), np.uint32)
    _check(lib.sfb_build_nt_lut(_np(nt), _np(layout), nb), "sfb_build_nt_lut")
    nt = np.ascontiguousarray(nt[:blocks])
    nn = np.zeros((nb + blocks, 2), np.uint32)
    nn_max = C.c_uint32(nn_max_init)
    _check(lib.sfb_build_nn_lut(_np(nn), _np(nt), blocks, nb, C.byref(nn_max)), "sfb_build_nn_lut")
    rblk = np.zeros((max(blocks, 1), 2), np.uint32)
    _check(lib.sfb_build_rblk_lut(_np(rblk), _np(nn), nb), "sfb_build_rblk_lut")
    order = np.zeros(nb, np.uint32)
    _check(lib.sfb_build_row_order(_np(order), _np(nn), nb), "sfb_build_row_order")
    return Luts(nt_lut=nt, nn_lut=nn, rblk_lut=np.ascontiguousarray(rblk[:blocks]), row_order=order,
                nn_max=int(nn_max.value), blocks=blocks, nb=nb)


def element_mask(nt_lut, bs, kind, local_attn_ctx=0):
    nt_lut = np.ascontiguousarray(nt_lut, np.uint32)
    blocks = nt_lut.shape[0]
    keep = np.zeros((blocks, bs, bs), np.uint8)
    _check(lib.sfb_element_mask(_np(keep), _np(nt_lut), blocks, bs, kind, local_attn_ctx),
           "sfb_element_mask")
    return keep


def pack_mask(keep):
    blocks, bs, _ = keep.shape
    words = np.zeros(blocks * bs, np.uint64 if bs == 64 else np.uint32)
    _check(lib.sfb_pack_mask(_np(words), _np(np.ascontiguousarray(keep, np.uint8)), blocks, bs),
           "sfb_pack_mask")
    return words


def transpose_mask(words, blocks, bs):
    out = np.zeros_like(words)
    _check(lib.sfb_transpose_mask(_np(out), _np(words), blocks, bs), "sfb_transpose_mask")
    return out


WORK_ITEM_DTYPE = np.dtype([(n, np.uint32) for n in
                            ("row", "first", "count", "nchunks", "chunk", "slot", "part", "reserved")])


def build_schedule(nn_lut, nb, max_blocks=16):
    """Work items of a scheduled fused launch: dict(items structured array, n_slots, n_parts)."""
    nn_lut = np.ascontiguousarray(nn_lut, np.uint32)
    n_items, n_slots, n_parts = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    _check(lib.sfb_build_schedule(None, C.byref(n_items), C.byref(n_slots), C.byref(n_parts),
                                  _np(nn_lut), nb, C.c_uint32(max_blocks)), "sfb_build_schedule")
    items = np.zeros(n_items.value, WORK_ITEM_DTYPE)
    _check(lib.sfb_build_schedule(_np(items), C.byref(n_items), C.byref(n_slots), C.byref(n_parts),
                                  _np(nn_lut), nb, C.c_uint32(max_blocks)), "sfb_build_schedule")
    return Luts(items=items, n_items=int(n_items.value), n_slots=int(n_slots.value),
                n_parts=int(n_parts.value))


def schedule_workspace_bytes(sched, batch, heads, block_size, d):
    return int(lib.sfb_schedule_workspace_bytes(C.c_uint32(sched["n_slots"]), C.c_uint32(sched["n_parts"]),
                                                C.c_uint32(batch), C.c_uint32(heads),
                                                C.c_uint32(block_size), C.c_uint32(d)))


def magicu64(d):
    m, s = C.c_uint32(0), C.c_uint32(0)
    lib.sfb_magicu64(C.c_uint32(d), C.byref(m), C.byref(s))
    return m.value, s.value


def device_available():
    return bool(lib.sfb_device_available())


# ------------------------------------------------------------------------------------ device ops
def to_device(array):
    """numpy descriptor -> device buffer (torch tensor of raw bytes; uint32/uint64 views are not needed)."""
    import torch
    raw = np.ascontiguousarray(array).view(np.uint8).reshape(-1)
    return torch.from_numpy(raw.copy()).cuda()


def _dtype_code(t):
    import torch
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise SfbError(5, "dtype of %s" % (t.dtype,))


def fused_attention(q, k, v, nn_lut, block_size, blocks, scale, mask=None, valid_len=None,
                    row_order=None, lut_heads=1, mask_heads=1, out=None):
    """O = block-sparse attention(q, k, v); q/k/v [B, L, H, d] fp32 or bf16 CUDA tensors, O fp32.

    nn_lut / mask / valid_len / row_order are device buffers (see to_device); mask is block-major."""
    import torch
    B, L, H, d = q.shape
    if out is None:
        out = torch.empty((B, L, H, d), dtype=torch.float32, device=q.device)
    nb = L // block_size
    for t in (q, k, v, out):
        if not t.is_contiguous():
            raise SfbError(4, "non-contiguous tensor")
    _check(lib.sfb_fused_attention(_stream(), _dev(q), _dev(k), _dev(v), _dev(out), _dtype_code(q),
                                   _dev(nn_lut), _dev(mask), _dev(valid_len), _dev(row_order),
                                   C.c_uint32(block_size), C.c_uint32(blocks), C.c_uint32(B),
                                   C.c_uint32(nb), C.c_uint32(H), C.c_uint32(d), C.c_uint32(lut_heads),
                                   C.c_uint32(nb + blocks), C.c_uint32(mask_heads), C.c_float(scale)),
           "sfb_fused_attention")
    return out


def fused_attention_scheduled(q, k, v, nn_lut, items, sched, workspace, block_size, blocks, scale,
                              mask=None, valid_len=None, mask_heads=1, out=None):
    """fused_attention over sfb_build_schedule's work items; `items` and `workspace` are device buffers
    (workspace: zero-filled uint8 tensor of schedule_workspace_bytes(), or None if nothing is split)."""
    import torch
    B, L, H, d = q.shape
    if out is None:
        out = torch.empty((B, L, H, d), dtype=torch.float32, device=q.device)
    nb = L // block_size
    for t in (q, k, v, out):
        if not t.is_contiguous():
            raise SfbError(4, "non-contiguous tensor")
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(lib.sfb_fused_attention_scheduled(
        _stream(), _dev(q), _dev(k), _dev(v), _dev(out), _dtype_code(q), _dev(nn_lut), _dev(mask),
        _dev(valid_len), _dev(items), C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_slots"]),
        C.c_uint32(sched["n_parts"]), _dev(workspace), C.c_size_t(ws_bytes), C.c_uint32(block_size),
        C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(nb), C.c_uint32(H), C.c_uint32(d),
        C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_attention_scheduled")
    return out


# ------------------------------------------------------------------------------------ unfused trio
def _torch_dtype(code):
    import torch
    return torch.bfloat16 if code == BF16 else torch.float32


def bst_sgemm_nt(lut, a, b, block_size, blocks, out_dtype=None, lut_heads=1, c=None):
    """sdd: S [B, H, blocks, bs, bs] = a_rowblk . b_colblk^T per NT-LUT entry (openai_blocksparse.h:202)."""
    import torch
    B, L, H, d = a.shape
    if c is None:
        c = torch.empty((B, H, blocks, block_size, block_size), device=a.device,
                        dtype=_torch_dtype(F32 if out_dtype is None else out_dtype))
    _check(lib.sfb_sdd_nt(_stream(), _dev(lut), _dev(a), _dev(b), _dev(c), _dtype_code(a), _dtype_code(c),
                          C.c_uint32(block_size), C.c_uint32(blocks), C.c_uint32(B),
                          C.c_uint32(L // block_size), C.c_uint32(b.shape[1] // block_size), C.c_uint32(H),
                          C.c_uint32(d), C.c_uint32(lut_heads), C.c_uint32(blocks)), "sfb_sdd_nt")
    return c


def BlocksparseMaskedSoftmax(lut, mask, x, ctx_blks, scale, out_dtype=None, valid_len=None, lut_heads=1,
                             mask_heads=1, max_lut=0, y=None):
    """Row softmax over the sparse scores (blocksparse.h:649); mask is ROW-major (transpose_mask)."""
    import torch
    B, H, blocks, bs, _ = x.shape
    if y is None:
        y = torch.empty_like(x, dtype=_torch_dtype(_dtype_code(x) if out_dtype is None else out_dtype))
    _check(lib.sfb_masked_softmax(_stream(), _dev(lut), _dev(mask), _dev(x), _dev(y), _dtype_code(x),
                                  _dtype_code(y), _dev(valid_len), C.c_uint32(bs), C.c_uint32(blocks),
                                  C.c_uint32(B), C.c_uint32(H), C.c_uint32(ctx_blks), C.c_uint32(lut_heads),
                                  C.c_uint32(ctx_blks + blocks), C.c_uint32(max_lut),
                                  C.c_uint32(mask_heads), C.c_float(scale)), "sfb_masked_softmax")
    return y


def bst_sgemm_xn(lut, a, b, ctx_blks_c, op=NN_OP, lut_heads=1, magic=1, shift=0, max_lut=0, c=None):
    """dsd: O [B, L, H, d] = sum_blk P_blk . V_colblk (blocksparse.h:965)."""
    import torch
    B, H, blocks, bs, _ = a.shape
    _, Lb, _, d = b.shape
    if c is None:
        c = torch.empty((B, ctx_blks_c * bs, H, d), device=b.device, dtype=torch.float32)
    _check(lib.sfb_dsd_xn(_stream(), _dev(lut), _dev(a), _dev(b), _dev(c), _dtype_code(a), _dtype_code(b),
                          C.c_uint32(bs), C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(Lb // bs),
                          C.c_uint32(ctx_blks_c), C.c_uint32(H), C.c_uint32(d), C.c_uint32(lut_heads),
                          C.c_uint32(ctx_blks_c + blocks), C.c_uint32(op), C.c_uint32(magic),
                          C.c_uint32(shift), C.c_uint32(max_lut)), "sfb_dsd_xn")
    return c


def fusion_attention2(nn_lut, a, b, block_size, blocks, scale, mask=None, valid_len=None, out_dtype=None,
                      lut_heads=1, mask_heads=1, y=None):
    """sdd + masked softmax in one kernel -> P (fusion_blocksparse.h:1212); mask is BLOCK-major."""
    import torch
    B, L, H, d = a.shape
    if y is None:
        y = torch.empty((B, H, blocks, block_size, block_size), device=a.device,
                        dtype=_torch_dtype(F32 if out_dtype is None else out_dtype))
    nb = L // block_size
    _check(lib.sfb_fused_sdd_softmax(_stream(), _dev(nn_lut), _dev(a), _dev(b), _dev(y), _dtype_code(a),
                                     _dtype_code(y), _dev(mask), _dev(valid_len), C.c_uint32(block_size),
                                     C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(nb), C.c_uint32(H),
                                     C.c_uint32(d), C.c_uint32(lut_heads), C.c_uint32(nb + blocks),
                                     C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_sdd_softmax")
    return y


fusion_attention1 = fusion_attention2
