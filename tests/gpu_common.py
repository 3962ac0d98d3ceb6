"""Shared helpers of the GPU parity tests: seeded inputs, oracle runs, error metrics."""
import numpy as np
import torch

import oracle_lib as orc
from sfb import sfb

TOL_F32 = 1e-4   # max |gpu - oracle| / max |oracle| for fp32 inputs
TOL_BF16 = 1e-2  # the same for bf16 inputs (oracle run in fp32 on the bf16-rounded inputs)


def rel_err(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def elementwise_err(got, want, floor):
    """max over elements of |diff| / max(|want|, floor)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float((np.abs(got - want) / np.maximum(np.abs(want), floor)).max())


def qkv(B, L, H, d, seed, bf16=False):
    out = [orc.fill_normal((B, L, H, d), seed + i) for i in range(3)]
    if bf16:
        out = [orc.round_bf16(x) for x in out]
    return out


def dev(x, bf16=False):
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t.to(torch.bfloat16) if bf16 else t


PATTERNS = {
    "local": lambda nb: sfb.layout_local(nb, 1, bidirectional=True),
    "local_causal": lambda nb: sfb.layout_local(nb, 1),
    "fixed": lambda nb: sfb.layout_fixed(1, nb, 4, causal=False)[0],
    "strided": lambda nb: sfb.layout_strided(nb, 4, 4),
    "bigbird": lambda nb: sfb.layout_bigbird(nb, 1, 2, True, sfb.bigbird_draw(nb, 1, 2, True, 3, 1234)),
    "full": lambda nb: sfb.layout_full(nb, causal=False),
    "causal": lambda nb: sfb.layout_full(nb, causal=True),
}


def run_fused(Q, K, V, luts, bs, scale, bf16=False, mask=None, valid_len=None, use_order=True,
              lut_heads=1, mask_heads=1, nn_lut=None, blocks=None, max_blocks=None, workspace=None):
    """max_blocks != None runs the scheduled entry point (rows longer than max_blocks are split)."""
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    nn = sfb.to_device(luts["nn_lut"] if nn_lut is None else nn_lut)
    m = None if mask is None else sfb.to_device(mask)
    vl = None if valid_len is None else sfb.to_device(np.asarray(valid_len, np.int32))
    if max_blocks is not None:
        B, L, H, d = Q.shape
        sched = sfb.build_schedule(luts["nn_lut"], L // bs, max_blocks)
        if workspace is None:
            nbytes = sfb.schedule_workspace_bytes(sched, B, H, bs, d)
            workspace = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device="cuda")
        o = sfb.fused_attention_scheduled(q, k, v, nn, sfb.to_device(sched["items"]), sched, workspace, bs,
                                          luts["blocks"], scale, mask=m, valid_len=vl,
                                          mask_heads=mask_heads)
        torch.cuda.synchronize()
        assert int(workspace[:max(4 * B * H * sched["n_slots"], 4)].view(torch.int32).abs().sum()) == 0, \
            "arrival counters must be left at zero"
        return o.cpu().numpy()
    order = sfb.to_device(luts["row_order"]) if use_order else None
    o = sfb.fused_attention(q, k, v, nn, bs, luts["blocks"] if blocks is None else blocks, scale,
                            mask=m, valid_len=vl, row_order=order, lut_heads=lut_heads,
                            mask_heads=mask_heads)
    torch.cuda.synchronize()
    return o.cpu().numpy()
