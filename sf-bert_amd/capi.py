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
    # torch ships its own copy of the HIP runtime; it has to be in the process before this library is
    # loaded, so that both resolve to the same runtime and torch's streams are valid for our launches
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
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
lib.sfb_scale_parts.restype = None
lib.sfb_schedule_workspace_bytes.restype = C.c_size_t
lib.sfb_encoder_layer_workspace_bytes.restype = C.c_size_t
lib.sfb_suggest_max_blocks.restype = C.c_uint32
lib.sfb_model_workspace_bytes.restype = C.c_size_t
lib.sfb_split_softmax_scratch_bytes.restype = C.c_size_t
lib.sfb_backward_workspace_bytes.restype = C.c_size_t
lib.sfb_dsd_workspace_bytes.restype = C.c_size_t
lib.sfb_resident_work_groups.restype = C.c_uint32
lib.sfb_resident_work_groups_for.restype = C.c_uint32
lib.sfb_stream_workspace_bytes.restype = C.c_size_t
lib.sfb_static_scratch_bytes.restype = C.c_size_t
lib.sfb_gemm_release.restype = None

#: every symbol include/sfbert_hip.h declares (checked by the CPU test-suite)
EXPORTED = [
    "sfb_status_string", "sfb_device_available",
    "sfb_layout_full", "sfb_layout_local", "sfb_layout_fixed", "sfb_layout_strided_chunks",
    "sfb_layout_strided", "sfb_layout_bigbird", "sfb_bigbird_draw", "sfb_count_blocks",
    "sfb_build_nt_lut", "sfb_build_nn_lut", "sfb_build_rblk_lut", "sfb_build_tn_lut", "sfb_magicu64", "sfb_element_mask",
    "sfb_pack_mask", "sfb_transpose_mask", "sfb_build_row_order",
    "sfb_build_schedule", "sfb_build_schedule_heads", "sfb_suggest_max_blocks", "sfb_schedule_workspace_bytes",
    "sfb_build_stream", "sfb_stream_workspace_bytes", "sfb_stream_status", "sfb_stream_reset", "sfb_resident_work_groups",
    "sfb_resident_work_groups_for", "sfb_scale_parts", "sfb_gemm_tuning",
    "sfb_fused_attention_streamed",
    "sfb_static_scratch_bytes", "sfb_fused_attention_scheduled_noalloc",
    "sfb_fused_attention", "sfb_fused_attention_scheduled", "sfb_fused_attention_scheduled_to",
    "sfb_fused_attention_scheduled_strided", "sfb_fused_attention_scheduled_heads",
    "sfb_fused_attention_scheduled_lse", "sfb_fused_attention_backward", "sfb_backward_workspace_bytes",
    "sfb_sdd_nt", "sfb_masked_softmax", "sfb_masked_softmax_grad", "sfb_dsd_xn", "sfb_dsd_xn_scheduled",
    "sfb_dsd_workspace_bytes", "sfb_fused_sdd_softmax",
    "sfb_split_softmax_scratch_bytes", "sfb_fused_sdd_softmax_split", "sfb_row_dot", "sfb_sdd_softmax_grad",
    "sfb_bias_act", "sfb_layernorm", "sfb_bias_residual_layernorm", "sfb_add_matrix", "sfb_transpose_0213", "sfb_embedding_lookup", "sfb_cast_f32_bf16",
    "sfb_pack_qkv", "sfb_gemm_release", "sfb_gemm", "sfb_gemm_bias", "sfb_gemm_bias_gelu", "sfb_gemm_bias_gelu_scaled", "sfb_encoder_layer_workspace_bytes", "sfb_encoder_layer_forward",
    "sfb_encoder_layer_forward_streamed",
    "sfb_encoder_layer_forward_pre_ln", "sfb_gemm_nt", "sfb_softmax_cross_entropy", "sfb_model_workspace_bytes",
    "sfb_model_forward",
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
    """nt_lut [blocks,2], nn_lut / tn_lut [nb+blocks,2], rblk_lut [blocks,2], row_order [nb], nn_max, tn_max,
    blocks, nb."""
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
    tn = np.zeros((nb + blocks, 2), np.uint32)
    tn_max = C.c_uint32(0)
    _check(lib.sfb_build_tn_lut(_np(tn), _np(nt), blocks, nb, C.byref(tn_max)), "sfb_build_tn_lut")
    return Luts(nt_lut=nt, nn_lut=nn, tn_lut=tn, rblk_lut=np.ascontiguousarray(rblk[:blocks]), row_order=order,
                nn_max=int(nn_max.value), tn_max=int(tn_max.value), blocks=blocks, nb=nb)


def element_mask(nt_lut, bs, kind, local_attn_ctx=0):
    nt_lut = np.ascontiguousarray(nt_lut, np.uint32)
    blocks = nt_lut.shape[0]
    keep = np.zeros((blocks, bs, bs), np.uint8)
    _check(lib.sfb_element_mask(_np(keep), _np(nt_lut), blocks, bs, kind, local_attn_ctx),
           "sfb_element_mask")
    return keep


def pack_mask(keep):
    blocks, bs, _ = keep.shape
    words = np.zeros(blocks * bs, {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}.get(bs, np.uint32))
    _check(lib.sfb_pack_mask(_np(words), _np(np.ascontiguousarray(keep, np.uint8)), blocks, bs),
           "sfb_pack_mask")
    return words


def transpose_mask(words, blocks, bs):
    out = np.zeros_like(words)
    _check(lib.sfb_transpose_mask(_np(out), _np(words), blocks, bs), "sfb_transpose_mask")
    return out


WORK_ITEM_DTYPE = np.dtype([(n, np.uint32) for n in
                            ("row", "first", "count", "nchunks", "chunk", "slot", "part", "lut_first")])


def suggest_max_blocks(nn_lut, nb, batch_heads):
    """Chunk length for build_schedule that suits a launch over batch_heads (batch, head) pairs."""
    nn_lut = np.ascontiguousarray(nn_lut, np.uint32)
    return int(lib.sfb_suggest_max_blocks(_np(nn_lut), nb, C.c_uint32(batch_heads)))


def build_schedule(nn_lut, nb, max_blocks=16):
    """Work items of a scheduled fused launch: dict(items structured array, n_slots, n_parts)."""
    nn_lut = np.ascontiguousarray(nn_lut, np.uint32)
    n_items, n_heavy, n_slots, n_parts = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    _check(lib.sfb_build_schedule(None, C.byref(n_items), C.byref(n_heavy), C.byref(n_slots), C.byref(n_parts),
                                  _np(nn_lut), nb, C.c_uint32(max_blocks)), "sfb_build_schedule")
    items = np.zeros(n_items.value, WORK_ITEM_DTYPE)
    _check(lib.sfb_build_schedule(_np(items), C.byref(n_items), C.byref(n_heavy), C.byref(n_slots),
                                  C.byref(n_parts), _np(nn_lut), nb, C.c_uint32(max_blocks)), "sfb_build_schedule")
    return Luts(items=items, n_items=int(n_items.value), n_heavy=int(n_heavy.value),
                n_slots=int(n_slots.value), n_parts=int(n_parts.value))


WORK_ITEM_SKIP = 0xFFFFFFFF


def build_schedule_heads(nn_lut, nb, lut_heads, max_blocks=16):
    """sfb_build_schedule_heads: one work-item list per head for lut_heads look-up tables of equal length
    concatenated; dict(items structured array [lut_heads][n_items] (short lists filled with WORK_ITEM_SKIP rows),
    n_items, n_heavy, n_slots, n_parts, lut_heads, lut_dim)."""
    nn_lut = np.ascontiguousarray(nn_lut, np.uint32)
    lut_dim = nn_lut.reshape(-1, 2).shape[0] // lut_heads
    n_items, n_heavy, n_slots, n_parts = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    args = (C.byref(n_items), C.byref(n_heavy), C.byref(n_slots), C.byref(n_parts), _np(nn_lut), nb,
            C.c_uint32(lut_heads), C.c_uint32(lut_dim), C.c_uint32(max_blocks))
    _check(lib.sfb_build_schedule_heads(None, *args), "sfb_build_schedule_heads")
    items = np.zeros((lut_heads, n_items.value), WORK_ITEM_DTYPE)
    _check(lib.sfb_build_schedule_heads(_np(items), *args), "sfb_build_schedule_heads")
    return Luts(items=items, n_items=int(n_items.value), n_heavy=int(n_heavy.value), n_slots=int(n_slots.value),
                n_parts=int(n_parts.value), lut_heads=int(lut_heads), lut_dim=int(lut_dim))


def fused_attention_scheduled_heads(q, k, v, nn_lut, items, sched, workspace, block_size, blocks, scale, mask=None,
                                    valid_len=None, mask_heads=1, out=None, lse=None):
    """sfb_fused_attention_scheduled_heads over build_schedule_heads()'s per-head work items."""
    import torch
    B, L, H, d = q.shape
    if out is None:
        out = torch.empty((B, L, H, d), dtype=torch.float32, device=q.device)
    for t in (q, k, v, out):
        if not t.is_contiguous():
            raise SfbError(4, "non-contiguous tensor")
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(lib.sfb_fused_attention_scheduled_heads(
        _stream(), _dev(q), _dev(k), _dev(v), _dev(out), _dev(lse), _dtype_code(q), _dtype_code(out), _dev(nn_lut),
        _dev(mask), _dev(valid_len), _dev(items), C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_heavy"]),
        C.c_uint32(sched["n_slots"]), C.c_uint32(sched["n_parts"]), _dev(workspace), C.c_size_t(ws_bytes),
        C.c_uint32(block_size), C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(L // block_size), C.c_uint32(H),
        C.c_uint32(d), C.c_uint32(sched["lut_heads"]), C.c_uint32(sched["lut_dim"]), C.c_uint32(mask_heads),
        C.c_float(scale)), "sfb_fused_attention_scheduled_heads")
    return out


def resident_work_groups(bf16=True, block_size=64, d=64, masked=False):
    """Work-groups the device keeps resident of the streamed kernel for these tensors (0 without a device)."""
    return int(lib.sfb_resident_work_groups_for(C.c_int(BF16 if bf16 else F32), C.c_uint32(block_size), C.c_uint32(d),
                                                C.c_int(1 if masked else 0)))


class StreamPlan(C.Structure):
    """sfb_stream_plan"""
    _fields_ = [(n, C.c_uint32) for n in ("wg_slots", "n_blocks", "n_items", "n_merges", "n_parts", "block_size",
                                          "batch_dim", "head_dim", "ctx_blks")] + [("balance", C.c_float), ("resident", C.c_uint32)] + \
               [(n, C.c_uint64) for n in ("slots_offset", "blocks_offset", "items_offset", "merges_offset",
                                          "total_bytes")]


STREAM_SLOT_DTYPE = np.dtype([(n, np.uint32) for n in ("block_begin", "n_blocks", "item_begin", "n_items",
                                                       "merge_begin", "n_merges", "reserved0", "reserved1")])
STREAM_BLOCK_DTYPE = np.dtype([(n, np.uint32) for n in ("kv_off", "info", "col", "q_off")])
STREAM_ITEM_DTYPE = np.dtype([(n, np.uint32) for n in ("q_off", "batch", "head", "row", "kind", "part", "lse_off",
                                                       "lut_first", "count", "first", "nchunks", "chunk", "r0", "r1",
                                                       "r2", "r3")])
STREAM_MERGE_DTYPE = np.dtype([(n, np.uint32) for n in ("q_off", "batch", "head", "row", "part", "nparts", "r0", "r1")])
STREAM_BLOCK_INDEX, STREAM_FIRST, STREAM_LAST = 0x0fffffff, 0x40000000, 0x80000000


def build_stream(nn_lut, nb, batch, heads, block_size, lut_heads=1, wg_slots=None, level=True, tail_percent=0,
                 d=64, bf16=True, masked=False):
    """Streams of key blocks for the resident work-groups of a streamed launch (sfb_build_stream): dict(plan
    (StreamPlan), blob (uint8 array to copy to the device), slots / blocks / items / merges (views of the blob),
    lut_heads, lut_dim).  nn_lut: one table, or lut_heads tables of equal length concatenated.  wg_slots None: what
    the device keeps resident of the kernel that a launch with head size d, bf16 or fp32 tensors and (masked) an
    element mask, key padding or log-sum-exp output runs (sfb_resident_work_groups_for)."""
    nn_lut = np.ascontiguousarray(nn_lut, np.uint32)
    lut_dim = nn_lut.shape[0] // lut_heads
    if wg_slots is None:
        wg_slots = resident_work_groups(bf16, block_size, d, masked) or 1024
    plan = StreamPlan()
    args = (_np(nn_lut), nb, C.c_uint32(lut_heads), C.c_uint32(lut_dim), C.c_uint32(batch), C.c_uint32(heads),
            C.c_uint32(block_size), C.c_uint32(wg_slots), C.c_int(1 if level else 0), C.c_uint32(tail_percent))
    _check(lib.sfb_build_stream(C.byref(plan), None, C.c_size_t(0), *args), "sfb_build_stream")
    blob = np.zeros(plan.total_bytes, np.uint8)
    _check(lib.sfb_build_stream(C.byref(plan), _np(blob), C.c_size_t(blob.nbytes), *args), "sfb_build_stream")

    def view(offset, count, dtype):
        return blob[offset:offset + count * dtype.itemsize].view(dtype)
    return Luts(plan=plan, blob=blob, lut_heads=int(lut_heads), lut_dim=int(lut_dim),
                slots=view(plan.slots_offset, plan.wg_slots, STREAM_SLOT_DTYPE),
                blocks=view(plan.blocks_offset, plan.n_blocks, STREAM_BLOCK_DTYPE),
                items=view(plan.items_offset, plan.n_items, STREAM_ITEM_DTYPE),
                merges=view(plan.merges_offset, plan.n_merges, STREAM_MERGE_DTYPE))


def gemm_tuning(level):
    """sfb_gemm_tuning: 0 = time the library's short list of GEMM kernels per problem, 1 = all that support it."""
    _check(lib.sfb_gemm_tuning(C.c_int(level)), "sfb_gemm_tuning")


def scale_parts(scale):
    """(pow2, rest) of sfb_scale_parts: scale * log2(e) = pow2 * rest."""
    a, b = C.c_float(0), C.c_float(0)
    lib.sfb_scale_parts(C.c_float(scale), C.byref(a), C.byref(b))
    return a.value, b.value


def stream_workspace_bytes(stream, d):
    return int(lib.sfb_stream_workspace_bytes(C.byref(stream["plan"]), C.c_uint32(d)))


def stream_status(stream, d, workspace):
    """0: every merge of the last launch found its records.  1: a bounded wait ran out; the workspace then holds
    stale flags and is cleared here (sfb_stream_reset), so that it can be used again."""
    status = int(lib.sfb_stream_status(C.byref(stream["plan"]), C.c_uint32(d), _dev(workspace)))
    if status == 1:
        stream_reset(stream, d, workspace)
    return status


def stream_reset(stream, d, workspace):
    _check(lib.sfb_stream_reset(_stream(), C.byref(stream["plan"]), C.c_uint32(d), _dev(workspace)), "sfb_stream_reset")


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


def fused_attention_forward_lse(q, k, v, nn_lut, items, sched, workspace, block_size, blocks, scale,
                                mask=None, valid_len=None, mask_heads=1):
    """Forward of a training step: (O fp32, lse [B, H, L]) through sfb_fused_attention_scheduled_lse."""
    import torch
    B, L, H, d = q.shape
    out = torch.empty((B, L, H, d), dtype=torch.float32, device=q.device)
    lse = torch.empty((B, H, L), dtype=torch.float32, device=q.device)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(lib.sfb_fused_attention_scheduled_lse(
        _stream(), _dev(q), _dev(k), _dev(v), _dev(out), _dev(lse), _dtype_code(q), F32, _dev(nn_lut), _dev(mask),
        _dev(valid_len), _dev(items), C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_heavy"]),
        C.c_uint32(sched["n_slots"]), C.c_uint32(sched["n_parts"]), _dev(workspace), C.c_size_t(ws_bytes),
        C.c_uint32(block_size), C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(L // block_size), C.c_uint32(H),
        C.c_uint32(d), C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_attention_scheduled_lse")
    return out, lse


def fused_attention_backward(q, k, v, o, d_out, lse, nn_lut, tn_lut, block_size, blocks, scale, mask=None,
                             valid_len=None, mask_heads=1, row_sched=None, col_sched=None, workspace=None,
                             lut_heads=1):
    """(dq, dk, dv) fp32 from bf16 or fp32 q, k, v, d_out (head sizes: multiples of 8 / 4 up to 128), the forward output o and lse, in two kernels
    (sfb_fused_attention_backward); nothing sparse goes through memory.  row_sched / col_sched: build_schedule()
    over the NN / TN look-up table with its "items" already on the device under "items_dev" (None: one
    work-group per block-row / block-column).  lut_heads = H: nn_lut / tn_lut hold one table per head (then without
    schedules)."""
    import torch
    B, L, H, d = q.shape
    dq, dk, dv = (torch.empty((B, L, H, d), dtype=torch.float32, device=q.device) for _ in range(3))
    delta = torch.empty((B, H, L), dtype=torch.float32, device=q.device)
    for t in (q, k, v, o, d_out):
        if not t.is_contiguous():
            raise SfbError(4, "non-contiguous tensor")
    rs, cs = row_sched or {}, col_sched or {}
    nbytes = int(lib.sfb_backward_workspace_bytes(C.c_uint32(rs.get("n_parts", 0)), C.c_uint32(cs.get("n_parts", 0)),
                                                  C.c_uint32(B), C.c_uint32(H), C.c_uint32(block_size), C.c_uint32(d)))
    if workspace is None and nbytes:
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    _check(lib.sfb_fused_attention_backward(
        _stream(), _dev(q), _dev(k), _dev(v), _dev(o), _dev(d_out), _dev(lse), _dev(delta), _dev(dq), _dev(dk),
        _dev(dv), _dtype_code(q), _dev(nn_lut), _dev(tn_lut), _dev(mask), _dev(valid_len),
        _dev(rs.get("items_dev")), C.c_uint32(rs.get("n_items", 0)), C.c_uint32(rs.get("n_heavy", 0)),
        C.c_uint32(rs.get("n_parts", 0)), _dev(cs.get("items_dev")), C.c_uint32(cs.get("n_items", 0)),
        C.c_uint32(cs.get("n_heavy", 0)), C.c_uint32(cs.get("n_parts", 0)), _dev(workspace),
        C.c_size_t(workspace.numel() if workspace is not None else 0), C.c_uint32(block_size), C.c_uint32(blocks),
        C.c_uint32(B), C.c_uint32(L // block_size), C.c_uint32(H), C.c_uint32(d), C.c_uint32(lut_heads),
        C.c_uint32(L // block_size + blocks), C.c_uint32(mask_heads), C.c_float(scale)),
        "sfb_fused_attention_backward")
    return dq, dk, dv


def fused_attention_scheduled(q, k, v, nn_lut, items, sched, workspace, block_size, blocks, scale,
                              mask=None, valid_len=None, mask_heads=1, out=None, out_dtype=F32):
    """fused_attention over sfb_build_schedule's work items; `items` and `workspace` are device buffers
    (workspace: zero-filled uint8 tensor of schedule_workspace_bytes(), or None if nothing is split).
    out_dtype BF16 (or a bf16 `out`) takes the sfb_fused_attention_scheduled_to entry point."""
    import torch
    B, L, H, d = q.shape
    if out is None:
        out = torch.empty((B, L, H, d), dtype=_torch_dtype(out_dtype), device=q.device)
    if out.dtype == torch.bfloat16:
        for t in (q, k, v, out):
            if not t.is_contiguous():
                raise SfbError(4, "non-contiguous tensor")
        ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
        _check(lib.sfb_fused_attention_scheduled_to(
            _stream(), _dev(q), _dev(k), _dev(v), _dev(out), _dtype_code(q), BF16, _dev(nn_lut), _dev(mask),
            _dev(valid_len), _dev(items), C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_heavy"]),
            C.c_uint32(sched["n_slots"]), C.c_uint32(sched["n_parts"]), _dev(workspace), C.c_size_t(ws_bytes),
            C.c_uint32(block_size), C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(L // block_size), C.c_uint32(H),
            C.c_uint32(d), C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_attention_scheduled_to")
        return out
    nb = L // block_size
    for t in (q, k, v, out):
        if not t.is_contiguous():
            raise SfbError(4, "non-contiguous tensor")
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(lib.sfb_fused_attention_scheduled(
        _stream(), _dev(q), _dev(k), _dev(v), _dev(out), _dtype_code(q), _dev(nn_lut), _dev(mask),
        _dev(valid_len), _dev(items), C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_heavy"]),
        C.c_uint32(sched["n_slots"]),
        C.c_uint32(sched["n_parts"]), _dev(workspace), C.c_size_t(ws_bytes), C.c_uint32(block_size),
        C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(nb), C.c_uint32(H), C.c_uint32(d),
        C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_attention_scheduled")
    return out


def fused_attention_scheduled_strided(qkv, nn_lut, items, sched, workspace, block_size, blocks, scale, heads,
                                      mask=None, valid_len=None, mask_heads=1, out_dtype=F32):
    """sfb_fused_attention_scheduled_strided on one [B, L, 3 * H * d] tensor holding Q | K | V side by side in every
    token row (the result of a merged projection)."""
    import torch
    B, L, width = qkv.shape
    d = width // (3 * heads)
    if not qkv.is_contiguous() or width != 3 * heads * d:
        raise SfbError(4, "qkv must be a contiguous [B, L, 3 * heads * d] tensor")
    out = torch.empty((B, L, heads, d), dtype=_torch_dtype(out_dtype), device=qkv.device)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    esz = qkv.element_size()
    base = qkv.data_ptr()
    _check(lib.sfb_fused_attention_scheduled_strided(
        _stream(), C.c_void_p(base), C.c_void_p(base + heads * d * esz), C.c_void_p(base + 2 * heads * d * esz),
        _dev(out), _dtype_code(qkv), out_dtype, _dev(nn_lut), _dev(mask), _dev(valid_len), _dev(items),
        C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_heavy"]), C.c_uint32(sched["n_slots"]),
        C.c_uint32(sched["n_parts"]), _dev(workspace), C.c_size_t(ws_bytes), C.c_uint32(block_size),
        C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(L // block_size), C.c_uint32(heads), C.c_uint32(d),
        C.c_uint32(width), C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_attention_scheduled_strided")
    return out


# ------------------------------------------------------------------------------------ unfused trio
def fused_attention_streamed(q, k, v, nn_lut, blob_dev, stream, workspace, block_size, blocks, scale, mask=None,
                             valid_len=None, mask_heads=1, out=None, lse=None):
    """sfb_fused_attention_streamed: resident work-groups walking build_stream()'s streams.  blob_dev: device copy
    of stream["blob"]; workspace: zero-filled uint8 tensor of stream_workspace_bytes(stream, d) bytes."""
    import torch
    B, L, H, d = q.shape
    if out is None:
        out = torch.empty((B, L, H, d), device=q.device, dtype=torch.float32)
    _check(lib.sfb_fused_attention_streamed(
        _stream(), _dev(q), _dev(k), _dev(v), _dev(out), _dev(lse), _dtype_code(q), _dtype_code(out), _dev(nn_lut),
        _dev(mask), _dev(valid_len), C.byref(stream["plan"]), _dev(blob_dev), _dev(workspace),
        C.c_size_t(workspace.numel()), C.c_uint32(block_size), C.c_uint32(blocks),
        C.c_uint32(B), C.c_uint32(L // block_size), C.c_uint32(H), C.c_uint32(d), C.c_uint32(stream["lut_heads"]),
        C.c_uint32(stream["lut_dim"]), C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_attention_streamed")
    return out


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


def BlocksparseMaskedSoftmaxGrad(lut, dy, y, ctx_blks, scale, lut_heads=1, max_lut=0, dx=None):
    """dx = (dy - sum_k dy*y) * y * scale over each sparse row (blocksparse.h:1164); dy, y, dx share a dtype."""
    import torch
    B, H, blocks, bs, _ = y.shape
    if dy.dtype != y.dtype or dy.shape != y.shape:
        raise SfbError(4, "dy and y differ in dtype or shape")
    if dx is None:
        dx = torch.empty_like(y)
    _check(lib.sfb_masked_softmax_grad(_stream(), _dev(lut), _dev(dy), _dev(y), _dev(dx), _dtype_code(y),
                                       C.c_uint32(bs), C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(H),
                                       C.c_uint32(ctx_blks), C.c_uint32(lut_heads), C.c_uint32(ctx_blks + blocks),
                                       C.c_uint32(max_lut), C.c_float(scale)), "sfb_masked_softmax_grad")
    return dx


def bst_sgemm_xn(lut, a, b, ctx_blks_c, op=NN_OP, lut_heads=1, magic=1, shift=0, max_lut=0, c=None):
    """dsd (blocksparse.h:965).  NN_OP: C [B, L, H, d] = sum_blk A_blk . B_colblk over each block-row (lut = NN
    LUT).  TN_OP: C = sum_blk A_blk^T . B_rowblk over each block-column (lut = TN LUT)."""
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


def dsd_workspace_bytes(sched, batch, heads, block_size, d):
    return int(lib.sfb_dsd_workspace_bytes(C.c_uint32(sched["n_parts"]), C.c_uint32(batch), C.c_uint32(heads),
                                           C.c_uint32(block_size), C.c_uint32(d)))


def bst_sgemm_xn_scheduled(lut, a, b, ctx_blks_c, items, sched, workspace, op=NN_OP, lut_heads=1, c=None):
    """sfb_dsd_xn_scheduled: bst_sgemm_xn launched over the work items of build_schedule(lut) (or
    build_schedule_heads with a table per head); workspace: device bytes, dsd_workspace_bytes() of them, or None
    when no line is cut."""
    import torch
    B, H, blocks, bs, _ = a.shape
    _, Lb, _, d = b.shape
    if c is None:
        c = torch.empty((B, ctx_blks_c * bs, H, d), device=b.device, dtype=torch.float32)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(lib.sfb_dsd_xn_scheduled(_stream(), _dev(lut), _dev(a), _dev(b), _dev(c), _dtype_code(a), _dtype_code(b),
                                    _dev(items), C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_heavy"]),
                                    C.c_uint32(sched["n_parts"]), _dev(workspace), C.c_size_t(ws_bytes),
                                    C.c_uint32(bs), C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(Lb // bs),
                                    C.c_uint32(ctx_blks_c), C.c_uint32(H), C.c_uint32(d), C.c_uint32(lut_heads),
                                    C.c_uint32(ctx_blks_c + blocks), C.c_uint32(op)), "sfb_dsd_xn_scheduled")
    return c


def fusion_attention2(nn_lut, a, b, block_size, blocks, scale, mask=None, valid_len=None, out_dtype=None,
                      lut_heads=1, mask_heads=1, y=None, row_order=None):
    """sdd + masked softmax in one kernel -> P (fusion_blocksparse.h:1212); mask is BLOCK-major; row_order:
    device buffer of build_luts()["row_order"] (longest block-rows first) or None."""
    import torch
    B, L, H, d = a.shape
    if y is None:
        y = torch.empty((B, H, blocks, block_size, block_size), device=a.device,
                        dtype=_torch_dtype(F32 if out_dtype is None else out_dtype))
    nb = L // block_size
    _check(lib.sfb_fused_sdd_softmax(_stream(), _dev(nn_lut), _dev(a), _dev(b), _dev(y), _dtype_code(a),
                                     _dtype_code(y), _dev(mask), _dev(valid_len), _dev(row_order), C.c_uint32(block_size),
                                     C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(nb), C.c_uint32(H),
                                     C.c_uint32(d), C.c_uint32(lut_heads), C.c_uint32(nb + blocks),
                                     C.c_uint32(mask_heads), C.c_float(scale)), "sfb_fused_sdd_softmax")
    return y


fusion_attention1 = fusion_attention2


def fusion_attention2_split(nt_lut, nn_lut, a, b, block_size, blocks, scale, mask=None, valid_len=None,
                            out_dtype=None, lut_heads=1, mask_heads=1, y=None, scratch=None, spin_limit=1 << 16):
    """sdd + masked softmax -> P by one work-group per block with flag / spin exchange between the blocks of a
    block-row (the reference's fusion_nt_softmax2 decomposition; comparison variant).  Returns (P, status) where
    status is a device uint32 tensor: 0 = every block written."""
    import torch
    B, L, H, d = a.shape
    nb = L // block_size
    if y is None:
        y = torch.empty((B, H, blocks, block_size, block_size), device=a.device,
                        dtype=_torch_dtype(F32 if out_dtype is None else out_dtype))
    nbytes = int(lib.sfb_split_softmax_scratch_bytes(C.c_uint32(block_size), C.c_uint32(blocks), C.c_uint32(B),
                                                     C.c_uint32(H), C.c_uint32(nb)))
    if scratch is None:
        scratch = torch.empty(nbytes, dtype=torch.uint8, device=a.device)
    _check(lib.sfb_fused_sdd_softmax_split(_stream(), _dev(nt_lut), _dev(nn_lut), _dev(a), _dev(b), _dev(y),
                                           _dtype_code(a), _dtype_code(y), _dev(mask), _dev(valid_len), _dev(scratch),
                                           C.c_size_t(scratch.numel()), C.c_uint32(spin_limit), C.c_uint32(block_size),
                                           C.c_uint32(blocks), C.c_uint32(B), C.c_uint32(nb), C.c_uint32(H),
                                           C.c_uint32(d), C.c_uint32(lut_heads), C.c_uint32(mask_heads),
                                           C.c_float(scale)), "sfb_fused_sdd_softmax_split")
    return y, scratch[nbytes - 256:nbytes - 252].view(torch.int32)


def row_dot(d_out, o):
    """delta [B, H, L] = sum_d dO * O (the row term of the softmax gradient, since O = P V)."""
    import torch
    B, L, H, d = d_out.shape
    delta = torch.empty((B, H, L), device=d_out.device, dtype=torch.float32)
    _check(lib.sfb_row_dot(_stream(), _dev(delta), _dev(d_out), _dev(o), _dtype_code(d_out), C.c_uint32(B),
                           C.c_uint32(L), C.c_uint32(H), C.c_uint32(d)), "sfb_row_dot")
    return delta


def sdd_softmax_grad(nt_lut, d_out, v, p, delta, block_size, blocks, scale, lut_heads=1, ds=None):
    """dS = (dO V^T - delta) * P * scale per block in one kernel (dP stays in registers)."""
    import torch
    B, L, H, d = d_out.shape
    if ds is None:
        ds = torch.empty_like(p)
    _check(lib.sfb_sdd_softmax_grad(_stream(), _dev(nt_lut), _dev(d_out), _dev(v), _dev(p), _dev(delta), _dev(ds),
                                    _dtype_code(d_out), _dtype_code(p), C.c_uint32(block_size), C.c_uint32(blocks),
                                    C.c_uint32(B), C.c_uint32(L // block_size), C.c_uint32(H), C.c_uint32(d),
                                    C.c_uint32(lut_heads), C.c_float(scale)), "sfb_sdd_softmax_grad")
    return ds


def dsd_schedules(luts, nb, batch, heads, block_size, d, max_blocks=16):
    """Work items and workspaces for the products of attention_backward launched over work items: one set over the
    NN table (block-rows: dQ) and one over the TN table (block-columns: dV, dK).  luts: build_luts() of one layout."""
    import torch
    out = {}
    for key in ("nn_lut", "tn_lut"):
        sched = build_schedule(luts[key], nb, max_blocks)
        nbytes = max(dsd_workspace_bytes(sched, batch, heads, block_size, d), 256)
        out[key] = dict(items=to_device(sched["items"]), sched=sched,
                        workspace=torch.empty(nbytes, dtype=torch.uint8, device="cuda"))
    return out


def attention_backward(q, k, v, d_out, p, luts_dev, block_size, blocks, scale, work_dtype=None, o=None, schedules=None):
    """Gradients of O = P V, P = masked softmax(scale * Q K^T) from the stored probabilities P, in the order of
    the reference's backward (transformer_attention_optimize.cu:924-965):
        dV = P^T dO (TN), dP = dO V^T (NT), dS = softmax grad, dK = dS^T Q (TN), dQ = dS K (NN).
    q, k, v, d_out [B, L, H, d]; p [B, H, blocks, bs, bs]; luts_dev: dict of device buffers nt_lut, nn_lut,
    tn_lut.  dP / dS use p's dtype unless work_dtype says otherwise.  o: the forward output O (fp32), optional; when
    given, dP and the softmax gradient are computed by one kernel (sdd_softmax_grad).  schedules: dsd_schedules() of
    the layout, optional; the three dsd products whose operands have one type are then launched over its work items
    (long block-rows and block-columns cut).  Returns (dq, dk, dv) fp32."""
    nb = q.shape[1] // block_size
    code = _dtype_code(p) if work_dtype is None else work_dtype

    def product(key, sparse, dense, op):
        if schedules is not None and sparse.dtype == dense.dtype:
            s = schedules[key]
            return bst_sgemm_xn_scheduled(luts_dev[key], sparse, dense, nb, s["items"], s["sched"], s["workspace"], op=op)
        return bst_sgemm_xn(luts_dev[key], sparse, dense, nb, op=op)

    dv = product("tn_lut", p, d_out, TN_OP)
    if o is not None:
        # with the forward output at hand the NT product and the softmax gradient are one kernel
        ds = sdd_softmax_grad(luts_dev["nt_lut"], d_out, v, p, row_dot(d_out, o), block_size, blocks, scale)
        return product("nn_lut", ds, k, NN_OP), product("tn_lut", ds, q, TN_OP), dv
    dp = bst_sgemm_nt(luts_dev["nt_lut"], d_out, v, block_size, blocks, out_dtype=code)
    if dp.dtype != p.dtype:
        p = p.to(dp.dtype)
    ds = BlocksparseMaskedSoftmaxGrad(luts_dev["nn_lut"], dp, p, nb, scale, dx=dp)
    dk = product("tn_lut", ds, q, TN_OP)
    dq = product("nn_lut", ds, k, NN_OP)
    return dq, dk, dv


# ------------------------------------------------------------------------------------ layer ops
def bias_act(x, bias=None, residual=None, act=0, out_dtype=F32, out=None):
    """out = act(x + bias[col]) + residual (bias: ewops.h:10, gelu: ewops.h:32, tensor_add_tensor: ewops.h:296)."""
    import torch
    cols = x.shape[-1]
    rows = x.numel() // cols
    if out is None:
        out = torch.empty(x.shape, device=x.device, dtype=_torch_dtype(out_dtype))
    _check(lib.sfb_bias_act(_stream(), _dev(out), _dtype_code(out), _dev(x), _dev(bias), _dev(residual),
                            int(act), C.c_uint64(rows), C.c_uint32(cols)), "sfb_bias_act")
    return out


def bias(x, b):
    return bias_act(x, bias=b)


def gelu(x):
    return bias_act(x, act=1)


def tensor_add_tensor(a, b):
    return bias_act(a, residual=b)


def layernorm(x, gain, beta, out_dtype=F32, return_stats=False):
    """layernorm.h:13-38; returns out (and mean, rstd)."""
    import torch
    state = x.shape[-1]
    rows = x.numel() // state
    out = torch.empty(x.shape, device=x.device, dtype=_torch_dtype(out_dtype))
    mean = torch.empty(rows, device=x.device) if return_stats else None
    rstd = torch.empty(rows, device=x.device) if return_stats else None
    _check(lib.sfb_layernorm(_stream(), _dev(out), _dtype_code(out), _dev(mean), _dev(rstd), _dev(x),
                             _dev(gain), _dev(beta), C.c_uint32(rows), C.c_uint32(state)), "sfb_layernorm")
    return (out, mean, rstd) if return_stats else out


def bias_residual_layernorm(x, bias, residual, gain, beta, with_bf16=False):
    """LayerNorm((x + bias) + residual) in one pass; returns out fp32 (and a bf16 copy)."""
    import torch
    state = x.shape[-1]
    rows = x.numel() // state
    out = torch.empty(x.shape, device=x.device, dtype=torch.float32)
    out16 = torch.empty(x.shape, device=x.device, dtype=torch.bfloat16) if with_bf16 else None
    _check(lib.sfb_bias_residual_layernorm(_stream(), _dev(out), _dev(out16), _dev(x), _dev(bias), _dev(residual),
                                           _dev(gain), _dev(beta), C.c_uint32(rows), C.c_uint32(state)),
           "sfb_bias_residual_layernorm")
    return (out, out16) if with_bf16 else out


def transpose_0123to0213(x):
    """[d0, d1, d2, d3] -> [d0, d2, d1, d3] (ewops.h:314-331), fp32 on the device."""
    import torch
    d0, d1, d2, d3 = x.shape
    out = torch.empty((d0, d2, d1, d3), dtype=torch.float32, device=x.device)
    _check(lib.sfb_transpose_0213(_stream(), _dev(out), _dev(x), C.c_uint32(d0), C.c_uint32(d1), C.c_uint32(d2),
                                  C.c_uint32(d3)), "sfb_transpose_0213")
    return out


def tensor_add_matrix(a, m):
    import torch
    out = torch.empty_like(a)
    _check(lib.sfb_add_matrix(_stream(), _dev(out), _dev(a), _dev(m), C.c_uint32(a.shape[0]),
                              C.c_uint64(m.numel())), "sfb_add_matrix")
    return out


def embedding_lookup(table, ids, pos=None):
    """out[t] = table[ids[t]] (+ pos[t % seq_len]); ids int32 [B, L]."""
    import torch
    vocab, state = table.shape
    out = torch.empty(tuple(ids.shape) + (state,), device=table.device, dtype=torch.float32)
    seq_len = ids.shape[-1]
    _check(lib.sfb_embedding_lookup(_stream(), _dev(out), _dev(table), _dev(ids), _dev(pos),
                                    C.c_uint64(ids.numel()), C.c_uint32(state), C.c_uint32(seq_len),
                                    C.c_uint32(vocab)), "sfb_embedding_lookup")
    return out


def cast_bf16(x):
    import torch
    out = torch.empty(x.shape, device=x.device, dtype=torch.bfloat16)
    _check(lib.sfb_cast_f32_bf16(_stream(), _dev(out), _dev(x), C.c_uint64(x.numel())), "sfb_cast_f32_bf16")
    return out


def gemm(a, w):
    """C[m, n] = a[m, k] @ w[k, n], fp32 or bf16 operands, fp32 result (cblas_sgemm call sites, transformer.cpp:516)."""
    import torch
    m, k = a.shape
    n = w.shape[1]
    c = torch.empty((m, n), device=a.device, dtype=torch.float32)
    _check(lib.sfb_gemm(_stream(), _dev(c), _dev(a), _dev(w), _dtype_code(a), C.c_uint32(m), C.c_uint32(n),
                        C.c_uint32(k)), "sfb_gemm")
    return c


def gemm_bias(a, w, bias, out_dtype=None):
    """C[m, n] = a[m, k] @ w[k, n] + bias[n] in one kernel; C in a's dtype unless out_dtype says otherwise."""
    import torch
    m, k = a.shape
    n = w.shape[1]
    code = _dtype_code(a) if out_dtype is None else out_dtype
    c = torch.empty((m, n), device=a.device, dtype=_torch_dtype(code))
    _check(lib.sfb_gemm_bias(_stream(), _dev(c), code, _dev(a), _dev(w), _dev(bias), _dtype_code(a), C.c_uint32(m),
                             C.c_uint32(n), C.c_uint32(k)), "sfb_gemm_bias")
    return c


def gemm_bias_gelu(a, w, bias, out_dtype=None):
    """C[m, n] = gelu(a[m, k] @ w[k, n] + bias[n]), sigmoid-form GELU (ewops.h:32-43), in one kernel."""
    import torch
    m, k = a.shape
    n = w.shape[1]
    code = _dtype_code(a) if out_dtype is None else out_dtype
    c = torch.empty((m, n), device=a.device, dtype=_torch_dtype(code))
    _check(lib.sfb_gemm_bias_gelu(_stream(), _dev(c), code, _dev(a), _dev(w), _dev(bias), _dtype_code(a),
                                  C.c_uint32(m), C.c_uint32(n), C.c_uint32(k)), "sfb_gemm_bias_gelu")
    return c


def gemm_bias_gelu_scaled(a, w, bias, out_dtype=None):
    """(C, scale) with C[m, n] = scale * gelu(a[m, k] @ w[k, n] + bias[n]); scale is 1 or 1.702 (see the header)."""
    import torch
    m, k = a.shape
    n = w.shape[1]
    code = _dtype_code(a) if out_dtype is None else out_dtype
    c = torch.empty((m, n), device=a.device, dtype=_torch_dtype(code))
    scratch = torch.empty((n,), device=a.device, dtype=torch.float32)
    scale = C.c_float(0.0)
    _check(lib.sfb_gemm_bias_gelu_scaled(_stream(), _dev(c), code, C.byref(scale), _dev(scratch), _dev(a), _dev(w),
                                         _dev(bias), _dtype_code(a), C.c_uint32(m), C.c_uint32(n), C.c_uint32(k)),
           "sfb_gemm_bias_gelu_scaled")
    return c, scale.value


def gemm_nt(a, w):
    """C[m, n] = a[m, k] @ w[n, k]^T (the tied-embedding logits, transformer_inference_part.cpp:236)."""
    import torch
    m, k = a.shape
    n = w.shape[0]
    c = torch.empty((m, n), device=a.device, dtype=torch.float32)
    _check(lib.sfb_gemm_nt(_stream(), _dev(c), _dev(a), _dev(w), _dtype_code(a), C.c_uint32(m), C.c_uint32(n),
                           C.c_uint32(k)), "sfb_gemm_nt")
    return c


def softmax_cross_entropy(logits, labels, want_grad=False, in_place=False):
    """(mean loss [1], row losses [rows][, softmax - onehot]) of ewops.h:233-261 over int32 labels."""
    import torch
    rows, vocab = logits.shape
    loss = torch.empty(1, device=logits.device, dtype=torch.float32)
    row_loss = torch.empty(rows, device=logits.device, dtype=torch.float32)
    d = (logits if in_place else torch.empty_like(logits)) if want_grad else None
    _check(lib.sfb_softmax_cross_entropy(_stream(), _dev(loss), _dev(row_loss), _dev(d), _dev(logits), _dev(labels),
                                         C.c_uint64(rows), C.c_uint32(vocab)), "sfb_softmax_cross_entropy")
    return (loss, row_loss, d) if want_grad else (loss, row_loss)


class LayerWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("wq", "wk", "wv", "wo", "w1", "w2", "bq", "bk", "bv", "bo", "b1", "b2",
                                          "ln1_g", "ln1_b", "ln2_g", "ln2_b", "wqkv", "bqkv")]


def _pack_qkv(c_weights, tensors, dtype, n):
    """Fills wqkv / bqkv of a LayerWeights from its wq, wk, wv, bq, bk, bv (sfb_pack_qkv); the new tensors are kept
    in `tensors`."""
    import torch
    w = tensors["wq"]
    tensors["wqkv"] = torch.empty((n, 3 * n), dtype=w.dtype, device=w.device)
    tensors["bqkv"] = torch.empty(3 * n, dtype=torch.float32, device=w.device)
    _check(lib.sfb_pack_qkv(_stream(), _dev(tensors["wqkv"]), _dev(tensors["bqkv"]), C.byref(c_weights), dtype,
                            C.c_uint32(n)), "sfb_pack_qkv")
    c_weights.wqkv, c_weights.bqkv = tensors["wqkv"].data_ptr(), tensors["bqkv"].data_ptr()


class EncoderLayer:
    """One post-LN encoder layer with block-sparse attention (sfb_encoder_layer_forward).

    weights: dict of fp32 CUDA tensors (wq..w2 [in, out], bq..b2, ln1_g, ln1_b, ln2_g, ln2_b);
    dtype BF16 casts the six matrices to bf16 once."""

    def __init__(self, weights, luts, block_size, heads, head_state, ffn, dtype=F32, max_blocks=16, pre_ln=False,
                 streamed=False, lut_heads=1, mask_heads=1, merge_qkv=True):
        """streamed: the attention runs over build_stream()'s streams (sfb_encoder_layer_forward_streamed); then
        luts["nn_lut"] may hold lut_heads tables (one per head) and the mask passed to forward() mask_heads masks.
        merge_qkv: Q, K and V as one product (used by layers whose attention is a scheduled launch)."""
        import torch
        self.dtype, self.bs, self.heads, self.d, self.ffn = dtype, block_size, heads, head_state, ffn
        self.luts = luts
        self.pre_ln = pre_ln   # True: the reference's own wiring (sfb_encoder_layer_forward_pre_ln)
        self.streamed, self.lut_heads, self.mask_heads = streamed, lut_heads, mask_heads
        self._streams = {}
        self.tensors = {}
        for name, t in weights.items():
            t = t.contiguous()
            if dtype == BF16 and name in ("wq", "wk", "wv", "wo", "w1", "w2"):
                t = cast_bf16(t)
            self.tensors[name] = t
        self.c_weights = LayerWeights(**{n: t.data_ptr() for n, t in self.tensors.items()})
        if merge_qkv:
            _pack_qkv(self.c_weights, self.tensors, dtype, heads * head_state)
        self.nn_lut = to_device(luts["nn_lut"])
        self.sched = build_schedule(luts["nn_lut"], luts["nb"], max_blocks) if max_blocks and not streamed else None
        self.items = to_device(self.sched["items"]) if self.sched else None
        self._ws = {}

    def _workspaces(self, B, L, device):
        import torch
        key = (B, L)
        if key not in self._ws:
            nbytes = int(lib.sfb_encoder_layer_workspace_bytes(C.c_uint32(B), C.c_uint32(L), C.c_uint32(self.heads),
                                                               C.c_uint32(self.d), C.c_uint32(self.ffn), self.dtype))
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
            aws = None
            if self.sched:
                aws = torch.zeros(max(schedule_workspace_bytes(self.sched, B, self.heads, self.bs, self.d), 256),
                                  dtype=torch.uint8, device=device)
            self._ws[key] = (ws, aws)
        return self._ws[key]

    def forward(self, x, B, L, mask=None, valid_len=None, out=None):
        import torch
        if out is None:
            out = torch.empty_like(x)
        ws, aws = self._workspaces(B, L, x.device)
        if self.streamed:
            import torch
            key = (B, mask is not None or valid_len is not None)   # the two kinds of launch run different kernels
            if key not in self._streams:
                st = build_stream(self.luts["nn_lut"], L // self.bs, B, self.heads, self.bs, lut_heads=self.lut_heads,
                                  level=False, d=self.d, bf16=self.dtype == BF16,
                                  masked=mask is not None or valid_len is not None)
                self._streams[key] = (st, to_device(st["blob"]),
                                    torch.zeros(stream_workspace_bytes(st, self.d), dtype=torch.uint8, device=x.device))
            st, blob, sws = self._streams[key]
            _check(lib.sfb_encoder_layer_forward_streamed(
                _stream(), _dev(out), _dev(x), C.byref(self.c_weights), self.dtype, C.c_int(1 if self.pre_ln else 0),
                _dev(self.nn_lut), _dev(mask), _dev(valid_len), C.byref(st["plan"]), _dev(blob), _dev(sws),
                C.c_size_t(sws.numel()), C.c_uint32(self.bs), C.c_uint32(self.luts["blocks"]), C.c_uint32(B),
                C.c_uint32(L // self.bs), C.c_uint32(self.heads), C.c_uint32(self.d), C.c_uint32(st["lut_heads"]),
                C.c_uint32(st["lut_dim"]), C.c_uint32(self.mask_heads), C.c_uint32(self.ffn), _dev(ws),
                C.c_size_t(ws.numel())), "sfb_encoder_layer_forward_streamed")
            return out
        s = self.sched
        entry = lib.sfb_encoder_layer_forward_pre_ln if self.pre_ln else lib.sfb_encoder_layer_forward
        _check(entry(
            _stream(), _dev(out), _dev(x), C.byref(self.c_weights), self.dtype, _dev(self.nn_lut), _dev(mask),
            _dev(valid_len), _dev(self.items), C.c_uint32(s["n_items"] if s else 0),
            C.c_uint32(s["n_heavy"] if s else 0), C.c_uint32(s["n_slots"] if s else 0), C.c_uint32(s["n_parts"] if s else 0), _dev(aws),
            C.c_size_t(aws.numel() if aws is not None else 0), C.c_uint32(self.bs), C.c_uint32(self.luts["blocks"]),
            C.c_uint32(B), C.c_uint32(L // self.bs), C.c_uint32(self.heads), C.c_uint32(self.d),
            C.c_uint32(self.ffn), _dev(ws), C.c_size_t(ws.numel())), "sfb_encoder_layer_forward")
        return out


class ModelWeights(C.Structure):
    _fields_ = [("tok_embed", C.c_void_p), ("pos_embed", C.c_void_p), ("tok_embed_bf16", C.c_void_p),
                ("layers", C.POINTER(LayerWeights)), ("n_layers", C.c_uint32)]


class Model:
    """Embedding + N encoder layers + tied-embedding logits + cross-entropy loss (sfb_model_forward), in the shape
    of transformer_inference_part.cpp:190-256.

    tok [vocab, state], pos [ctx, state] fp32 CUDA tensors; layers: list of weight dicts as for EncoderLayer."""

    def __init__(self, tok, pos, layers, luts, block_size, heads, head_state, ffn, dtype=F32, max_blocks=16,
                 pre_ln=True, merge_qkv=True):
        self.dtype, self.bs, self.heads, self.d, self.ffn, self.pre_ln = dtype, block_size, heads, head_state, ffn, pre_ln
        self.luts = luts
        self.tok, self.pos = tok.contiguous(), pos.contiguous()
        self.tok16 = cast_bf16(self.tok) if dtype == BF16 else None
        self.layer_tensors = []
        for weights in layers:
            tensors = {}
            for name, t in weights.items():
                t = t.contiguous()
                if dtype == BF16 and name in ("wq", "wk", "wv", "wo", "w1", "w2"):
                    t = cast_bf16(t)
                tensors[name] = t
            self.layer_tensors.append(tensors)
        self.c_layers = (LayerWeights * max(len(layers), 1))(
            *[LayerWeights(**{n: t.data_ptr() for n, t in tensors.items()}) for tensors in self.layer_tensors])
        if merge_qkv:
            for i, tensors in enumerate(self.layer_tensors):
                _pack_qkv(self.c_layers[i], tensors, dtype, heads * head_state)
        self.c_weights = ModelWeights(self.tok.data_ptr(), self.pos.data_ptr(),
                                      self.tok16.data_ptr() if self.tok16 is not None else None, self.c_layers,
                                      len(layers))
        self.nn_lut = to_device(luts["nn_lut"])
        self.sched = build_schedule(luts["nn_lut"], luts["nb"], max_blocks) if max_blocks else None
        self.items = to_device(self.sched["items"]) if self.sched else None
        self._ws = {}

    def forward(self, ids, labels=None, mask=None, valid_len=None, want_logits=False, want_hidden=False):
        """ids [B, L] int32; returns dict(loss [1] if labels given, logits, hidden)."""
        import torch
        B, L = ids.shape
        vocab, n = self.tok.shape
        key = (B, L)
        if key not in self._ws:
            nbytes = int(lib.sfb_model_workspace_bytes(C.c_uint32(B), C.c_uint32(L), C.c_uint32(self.heads),
                                                       C.c_uint32(self.d), C.c_uint32(self.ffn), C.c_uint32(vocab),
                                                       self.dtype))
            aws = None
            if self.sched:
                aws = torch.zeros(max(schedule_workspace_bytes(self.sched, B, self.heads, self.bs, self.d), 256),
                                  dtype=torch.uint8, device=ids.device)
            self._ws[key] = (torch.empty(nbytes, dtype=torch.uint8, device=ids.device), aws)
        ws, aws = self._ws[key]
        out = {}
        if labels is not None:
            out["loss"] = torch.empty(1, device=ids.device, dtype=torch.float32)
        if want_logits:
            out["logits"] = torch.empty((B * L, vocab), device=ids.device, dtype=torch.float32)
        if want_hidden:
            out["hidden"] = torch.empty((B * L, n), device=ids.device, dtype=torch.float32)
        s = self.sched
        _check(lib.sfb_model_forward(
            _stream(), _dev(out.get("loss")), _dev(out.get("logits")), _dev(out.get("hidden")), _dev(ids), _dev(labels),
            C.byref(self.c_weights), self.dtype, int(self.pre_ln), _dev(self.nn_lut), _dev(mask), _dev(valid_len),
            _dev(self.items), C.c_uint32(s["n_items"] if s else 0), C.c_uint32(s["n_heavy"] if s else 0),
            C.c_uint32(s["n_slots"] if s else 0), C.c_uint32(s["n_parts"] if s else 0), _dev(aws),
            C.c_size_t(aws.numel() if aws is not None else 0), C.c_uint32(self.bs), C.c_uint32(self.luts["blocks"]),
            C.c_uint32(B), C.c_uint32(L // self.bs), C.c_uint32(self.heads), C.c_uint32(self.d), C.c_uint32(self.ffn),
            C.c_uint32(vocab), _dev(ws), C.c_size_t(ws.numel())), "sfb_model_forward")
        return out
