"""sfb_fused_attention_scheduled_noalloc (arrival counters and partial records in the library's static device array)
against sfb_fused_attention_scheduled_to (the same in a caller's workspace), through the C ABI."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_common import PATTERNS, TOL_BF16, TOL_F32, dev, qkv, rel_err
from sfb import sfb

pytestmark = pytest.mark.gpu


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def both_entries(B, H, L, d, bs, pattern, max_blocks, bf16, seed, masked=False, out_bf16=False):
    nb = L // bs
    luts = sfb.build_luts(PATTERNS[pattern](nb))
    sched = sfb.build_schedule(luts["nn_lut"], nb, max_blocks)
    assert sched["n_parts"] > 0, "the case must cut rows, else no scratch is used"
    Q, K, V = qkv(B, L, H, d, seed=seed, bf16=bf16)
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    nn, items = sfb.to_device(luts["nn_lut"]), sfb.to_device(sched["items"])
    mask = valid = None
    mask_np = valid_np = None
    if masked:
        mask_np = sfb.pack_mask((np.random.default_rng(seed).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8))
        valid_np = np.array([L - 37 * (b % 3) for b in range(B)], np.int32)
        mask, valid = sfb.to_device(mask_np), sfb.to_device(valid_np)
    code_in = sfb.BF16 if bf16 else sfb.F32
    code_out = sfb.BF16 if out_bf16 else sfb.F32
    odt = torch.bfloat16 if out_bf16 else torch.float32
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    common = (C.c_uint32(bs), C.c_uint32(luts["blocks"]), C.c_uint32(B), C.c_uint32(nb), C.c_uint32(H), C.c_uint32(d),
              C.c_uint32(1), C.c_float(0.125))
    head = (stream, ptr(q), ptr(k), ptr(v))
    desc = (code_in, code_out, ptr(nn), ptr(mask), ptr(valid), ptr(items), C.c_uint32(sched["n_items"]),
            C.c_uint32(sched["n_heavy"]), C.c_uint32(sched["n_slots"]), C.c_uint32(sched["n_parts"]))
    need = sfb.schedule_workspace_bytes(sched, B, H, bs, d)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    want = torch.full((B, L, H, d), 3.0, device="cuda", dtype=odt)
    rc = sfb.lib.sfb_fused_attention_scheduled_to(*head, ptr(want), *desc, ptr(ws), C.c_size_t(need), *common)
    assert rc == 0, rc
    got = torch.full((B, L, H, d), 5.0, device="cuda", dtype=odt)
    before = torch.cuda.memory_allocated()
    rc = sfb.lib.sfb_fused_attention_scheduled_noalloc(*head, ptr(got), *desc, *common)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    oracle = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, mask=mask_np, valid_len=valid_np, nthreads=16)
    return got, want, oracle, need


def test_noalloc_entry_matches_the_workspace_entry_twice_in_a_row():
    assert sfb.lib.sfb_static_scratch_bytes() == 8 << 20
    # the benchmarked launch: BigBird B4 H12 L4096, global rows cut in two
    got, want, oracle, need = both_entries(4, 12, 4096, 64, 64, "bigbird", 37, True, seed=11)
    assert 0 < need <= sfb.lib.sfb_static_scratch_bytes()
    assert torch.equal(got, want)
    assert rel_err(got.cpu().numpy(), oracle) <= TOL_BF16
    # a smaller launch right after it finds the array as the first one left it: more chunks per row, fp32 tensors,
    # element mask and key padding, bf16 output
    got, want, oracle, _ = both_entries(2, 3, 1024, 64, 64, "bigbird", 3, False, seed=12, masked=True, out_bf16=True)
    assert torch.equal(got, want)
    assert rel_err(got.float().cpu().numpy(), oracle) <= TOL_BF16   # fp32 arithmetic, result rounded to bf16
    # and once more the other way round (larger after smaller), block size 32
    got, want, oracle, _ = both_entries(1, 4, 2048, 64, 32, "bigbird", 5, True, seed=13)
    assert torch.equal(got, want)
    assert rel_err(got.cpu().numpy(), oracle) <= TOL_BF16


def test_noalloc_entry_rejects_launches_beyond_its_scratch():
    B, H, L, d, bs = 16, 12, 4096, 64, 64
    nb = L // bs
    luts = sfb.build_luts(PATTERNS["bigbird"](nb))
    sched = sfb.build_schedule(luts["nn_lut"], nb, 8)
    assert sfb.schedule_workspace_bytes(sched, B, H, bs, d) > sfb.lib.sfb_static_scratch_bytes()
    x = torch.zeros(64, device="cuda")
    rc = sfb.lib.sfb_fused_attention_scheduled_noalloc(
        None, ptr(x), ptr(x), ptr(x), ptr(x), sfb.BF16, sfb.F32, ptr(x), None, None, ptr(x),
        C.c_uint32(sched["n_items"]), C.c_uint32(sched["n_heavy"]), C.c_uint32(sched["n_slots"]),
        C.c_uint32(sched["n_parts"]), C.c_uint32(bs), C.c_uint32(luts["blocks"]), C.c_uint32(B), C.c_uint32(nb),
        C.c_uint32(H), C.c_uint32(d), C.c_uint32(1), C.c_float(0.125))
    assert rc == 10
    assert b"static device array" in sfb.lib.sfb_status_string(rc)
