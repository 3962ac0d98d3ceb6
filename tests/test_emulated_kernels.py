"""The kernels of libsfbert_hip run from their own sources on the host model (tests/emu_lib.py), through the C ABI,
against the CPU oracle: small cases of every attention entry point, under several lane orders and both timings of
LDS-direct loads.  `pytest -m gpu --emulate` runs the whole GPU suite the same way (minutes per file); this file is
the selection that fits the CPU suite.  Same tolerances as on the device: fp32 <= 1e-4, bf16 <= 1e-2, relative to
the largest value of the result."""
import numpy as np
import pytest
import torch

import emu_lib
import oracle_lib as orc

TOL = {False: 1e-4, True: 1e-2}


@pytest.fixture(scope="module")
def E():
    # the binding allocates its outputs and workspaces "on the device of its inputs": here in guarded host memory
    with pytest.MonkeyPatch.context() as patch:
        mod = emu_lib.install(patch)
        yield mod
    emu_lib.configure()


def rel_err(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def inputs(B, L, H, d, seed, bf16, n=3):
    out = [orc.fill_normal((B, L, H, d), seed + i) for i in range(n)]
    return [orc.round_bf16(x) for x in out] if bf16 else out


def layout(E, nb):
    lay = E.layout_bigbird(nb, 1, 1, True, E.bigbird_draw(nb, 1, 1, True, 1, 3)).copy()
    lay[2] = 0   # a block-row without blocks
    return lay


def masks(E, luts, bs, L, B, seed):
    keep = (np.random.default_rng(seed).random((luts["blocks"], bs, bs)) < 0.8).astype(np.uint8)
    valid = np.array([L, L - bs - 5][:B], np.int32)
    return E.pack_mask(keep), valid


def dev(x, bf16=False):
    return emu_lib.tensor(x, bf16)


def zeros(nbytes):
    return emu_lib.empty((max(int(nbytes), 256),), torch.uint8, fill=0)


MODES = [(0, True), (1, False), (14, True), (21, False)]   # (lane order, LDS-direct loads land late)


def cases(shapes):
    """Block 64 / head 64 under every mode with bf16 tensors (LDS-direct loads, transposing reads) and two with fp32
    (tiles staged through registers); the other shapes under one mode each."""
    out = []
    for bs, d in shapes:
        for bf16 in (True, False):
            if (bs, d) == (64, 64):
                modes = MODES if bf16 else [MODES[0], MODES[3]]
            else:
                modes = [MODES[0] if bf16 else MODES[3]]
            out += [(bs, d, bf16, order, lazy) for order, lazy in modes]
    return out


@pytest.mark.parametrize("bs,d,bf16,order,lazy", cases([(64, 64), (32, 64), (64, 32), (32, 96), (64, 128), (64, 40), (32, 72)]))
def test_fused_forward_plain_scheduled_streamed(E, bs, d, bf16, order, lazy):
    """One work-group per row, work items with rows cut into chunks (arrival counters, partial records, merge) and
    resident work-groups walking streams, each without and with element mask and key padding.  d = 40 and 72: head
    sizes that are not multiples of 32 (the tiles' last slice is loaded short, the output rows are stored directly)."""
    emu_lib.configure(order=order, lazy_loads=lazy)
    nb, B, H = 5, 2, 2
    L = nb * bs
    luts = E.build_luts(layout(E, nb))
    mask, valid = masks(E, luts, bs, L, B, d)
    Q, K, V = inputs(B, L, H, d, 10 + d, bf16)
    scale = float(1.0 / np.sqrt(d))
    q, k, v = (dev(x, bf16) for x in (Q, K, V))
    nn = E.to_device(luts["nn_lut"])
    sched = E.build_schedule(luts["nn_lut"], nb, 2)
    assert sched["n_parts"] > 0
    items = E.to_device(sched["items"])
    for m, vl in ((None, None), (mask, valid)):
        want = orc.attention(Q, K, V, luts["nn_lut"], bs, scale, mask=m, valid_len=vl)
        md, vd = (None if m is None else E.to_device(m)), (None if vl is None else E.to_device(vl))
        got = E.fused_attention(q, k, v, nn, bs, luts["blocks"], scale, mask=md, valid_len=vd)
        assert rel_err(got.float().numpy(), want) <= TOL[bf16], ("plain", emu_lib.message())
        ws = zeros(E.schedule_workspace_bytes(sched, B, H, bs, d))
        for _ in range(2):   # the second launch finds the counters as the first left them
            got = E.fused_attention_scheduled(q, k, v, nn, items, sched, ws, bs, luts["blocks"], scale, mask=md, valid_len=vd)
            assert rel_err(got.float().numpy(), want) <= TOL[bf16], ("scheduled", emu_lib.message())
        assert (got.numpy()[:, 2 * bs:3 * bs] == 0).all()
        if True:
            stream = E.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=24, d=d, bf16=bf16, masked=m is not None)
            assert stream["plan"].n_parts > 0
            sw = zeros(E.stream_workspace_bytes(stream, d))
            blob = E.to_device(stream["blob"])
            for _ in range(2):
                got = E.fused_attention_streamed(q, k, v, nn, blob, stream, sw, bs, luts["blocks"], scale, mask=md, valid_len=vd)
                assert E.stream_status(stream, d, sw) == 0
                assert rel_err(got.float().numpy(), want) <= TOL[bf16], ("streamed", emu_lib.message())
    counts = emu_lib.counts()
    assert counts["mfma_bf16"][1] == 0 and counts["mfma_f32"][1] == 0 and counts["ds_read_tr16"][1] == 0, \
        "a matrix instruction or a transposing read ran with part of its wave"


def test_peaked_rows_take_the_general_loop(E):
    """Scores past 2^100 times the first block's offset: the lean bf16 loop notices and the row is redone by the loop
    that follows the maximum."""
    emu_lib.configure()
    bs, nb, B, H, d = 64, 4, 1, 2, 64
    luts = E.build_luts(layout(E, nb))
    Q, K, V = inputs(B, nb * bs, H, d, 91, True)
    Q = orc.round_bf16(Q * 8.0)
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 1.0)
    got = E.fused_attention(dev(Q, True), dev(K, True), dev(V, True), E.to_device(luts["nn_lut"]), bs, luts["blocks"], 1.0)
    assert rel_err(got.numpy(), want) <= TOL[True]


@pytest.mark.parametrize("bs,d,bf16,order,lazy", cases([(64, 64), (32, 32), (32, 96), (64, 128), (64, 40), (32, 72)]))
def test_fused_backward(E, bs, d, bf16, order, lazy):
    """dQ, dK, dV of the fused backward (whole lines, and lines cut into chunks with partial records) against the
    oracle's backward chain, without and with element mask and key padding.  d = 40 and 72: head sizes between the
    multiples of 32."""
    emu_lib.configure(order=order, lazy_loads=lazy)
    nb, B, H = 4, 2, 2
    L = nb * bs
    lay = layout(E, nb)
    lay[:, 3] = 0    # a block-column without blocks
    lay[3, 0] = 1
    luts = E.build_luts(lay)
    mask, valid = masks(E, luts, bs, L, B, d + 1)
    Q, K, V, dO = inputs(B, L, H, d, 30 + d, bf16, n=4)
    scale = float(1.0 / np.sqrt(d))
    q, k, v, do = (dev(x, bf16) for x in (Q, K, V, dO))
    nn, tn = E.to_device(luts["nn_lut"]), E.to_device(luts["tn_lut"])
    fwd = E.build_schedule(luts["nn_lut"], nb, 2)
    for m, vl in ((None, None), (mask, valid)):
        md, vd = (None if m is None else E.to_device(m)), (None if vl is None else E.to_device(vl))
        dQ, dK, dV, _ = orc.attention_backward(Q, K, V, dO, luts, bs, scale, mask=m, valid_len=vl)
        ws = zeros(E.schedule_workspace_bytes(fwd, B, H, bs, d))
        o, lse = E.fused_attention_forward_lse(q, k, v, nn, E.to_device(fwd["items"]), fwd, ws, bs, luts["blocks"], scale,
                                               mask=md, valid_len=vd)
        for max_blocks in (None, 2):
            rs = cs = None
            if max_blocks:
                rs, cs = E.build_schedule(luts["nn_lut"], nb, max_blocks), E.build_schedule(luts["tn_lut"], nb, max_blocks)
                rs["items_dev"], cs["items_dev"] = E.to_device(rs["items"]), E.to_device(cs["items"])
            dq, dk, dv = E.fused_attention_backward(q, k, v, o, do, lse, nn, tn, bs, luts["blocks"], scale, mask=md,
                                                    valid_len=vd, row_sched=rs, col_sched=cs)
            for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
                assert rel_err(got.numpy(), want) <= TOL[bf16], (name, max_blocks, emu_lib.message())
            assert (dq.numpy()[:, 2 * bs:3 * bs] == 0).all() and (dk.numpy()[:, 3 * bs:4 * bs] == 0).all()


@pytest.mark.parametrize("order,lazy", [MODES[0], MODES[2], MODES[3]])
@pytest.mark.parametrize("bs,d", [(64, 64), (32, 64), (64, 96), (64, 40), (32, 120)])
def test_unfused_sequence_bf16(E, bs, d, order, lazy):
    """sdd -> softmax -> dsd with bf16 tensors and bf16 S / P (at block 64, head 64: the streaming kernels with their
    counted waits and the ring-buffered dsd), the two-stage fusion, and the backward sequence."""
    emu_lib.configure(order=order, lazy_loads=lazy)
    nb, B, H = 6, 1, 2
    L = nb * bs
    luts = E.build_luts(layout(E, nb))
    blocks = luts["blocks"]
    scale = float(1.0 / np.sqrt(d))
    Q, K, V, dO = inputs(B, L, H, d, 50 + d, True, n=4)
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, scale)
    q, k, v, do = (dev(x, True) for x in (Q, K, V, dO))
    ld = {name: E.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    S = E.bst_sgemm_nt(ld["nt_lut"], q, k, bs, blocks, out_dtype=E.BF16)
    assert rel_err(S.float().numpy(), orc.sdd_nt(Q, K, luts["nt_lut"], bs)) <= TOL[True], emu_lib.message()
    p = E.BlocksparseMaskedSoftmax(ld["nn_lut"], None, S, nb, scale, out_dtype=E.BF16)
    assert rel_err(p.float().numpy(), P) <= TOL[True], emu_lib.message()
    p2 = E.fusion_attention2(ld["nn_lut"], q, k, bs, blocks, scale, out_dtype=E.BF16)
    assert rel_err(p2.float().numpy(), P) <= TOL[True], emu_lib.message()
    O = E.bst_sgemm_xn(ld["nn_lut"], p2, v, nb)
    assert rel_err(O.numpy(), orc.attention(Q, K, V, luts["nn_lut"], bs, scale)) <= TOL[True], emu_lib.message()
    dq, dk, dv = E.attention_backward(q, k, v, do, p2, ld, bs, blocks, scale, o=O)
    for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        assert rel_err(got.numpy(), want) <= 2e-2, (name, emu_lib.message())   # P, dP, dS each rounded to bf16 on the way


@pytest.mark.parametrize("bs,d", [(32, 64), (64, 64), (64, 36), (32, 100)])
def test_unfused_sequence_fp32(E, bs, d):
    emu_lib.configure()
    nb, B, H = 4, 1, 2
    luts = E.build_luts(layout(E, nb))
    blocks = luts["blocks"]
    Q, K, V, dO = inputs(B, nb * bs, H, d, 70, False, n=4)
    dQ, dK, dV, P = orc.attention_backward(Q, K, V, dO, luts, bs, 0.125)
    q, k, v, do = (dev(x) for x in (Q, K, V, dO))
    ld = {name: E.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    S = E.bst_sgemm_nt(ld["nt_lut"], q, k, bs, blocks)
    p = E.BlocksparseMaskedSoftmax(ld["nn_lut"], None, S, nb, 0.125)
    assert rel_err(p.numpy(), P) <= TOL[False], emu_lib.message()
    O = E.bst_sgemm_xn(ld["nn_lut"], p, v, nb)
    assert rel_err(O.numpy(), orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125)) <= TOL[False]
    dq, dk, dv = E.attention_backward(q, k, v, do, p, ld, bs, blocks, 0.125)
    for name, got, want in (("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        assert rel_err(got.numpy(), want) <= TOL[False], (name, emu_lib.message())


def test_scheduled_launch_with_one_table_per_head(E):
    """The reference's `fixed` pattern: one look-up table, one mask and one work-item list per head."""
    emu_lib.configure()
    bs, nb, B, H, d = 64, 8, 1, 4, 64
    lay = E.layout_fixed(H, nb, 4, causal=True)
    per_head = [E.build_luts(lay[h]) for h in range(H)]
    blocks = per_head[0]["blocks"]
    assert all(x["blocks"] == blocks for x in per_head)
    nn = np.concatenate([x["nn_lut"] for x in per_head])
    mask = np.concatenate([E.pack_mask(E.element_mask(x["nt_lut"], bs, E.MASK_CAUSAL_DIAG)) for x in per_head])
    sched = E.build_schedule_heads(nn, nb, H, 2)
    assert sched["n_parts"] > 0
    Q, K, V = inputs(B, nb * bs, H, d, 120, True)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    ws = zeros(E.schedule_workspace_bytes(sched, B, H, bs, d))
    want = orc.attention(Q, K, V, nn, bs, 0.125, mask=mask, lut_heads=H, mask_heads=H, blocks=blocks)
    got = E.fused_attention_scheduled_heads(q, k, v, E.to_device(nn), E.to_device(sched["items"]), sched, ws, bs, blocks,
                                            0.125, mask=E.to_device(mask), mask_heads=H).numpy()
    assert rel_err(got, want) <= TOL[True], emu_lib.message()


@pytest.mark.parametrize("tag,define", [("once", "SFB_TILE_LOAD_ONCE=1"), ("staged", "SFB_TILE_LOAD_STAGED=1")])
def test_tile_load_variants_of_the_bf16_loop(E, tag, define):
    """The two opt-in forms of the bf16 tile loads (one group of loads per tile with the steps in the instruction
    offsets; tiles staged through registers) give the same results as the default form, bit for bit, and agree with
    the oracle: plain and scheduled launches, lean and general loop."""
    variant = emu_lib.load(tag, (define,))
    bs, nb, B, H, d = 64, 5, 1, 2, 64
    luts = E.build_luts(layout(E, nb))
    mask, valid = masks(E, luts, bs, nb * bs, B, 5)
    Q, K, V = inputs(B, nb * bs, H, d, 140, True)
    q, k, v = (dev(x, True) for x in (Q, K, V))
    nn = E.to_device(luts["nn_lut"])
    sched = E.build_schedule(luts["nn_lut"], nb, 2)
    items = E.to_device(sched["items"])
    for order, lazy in (MODES[2],):
        emu_lib.configure(order=order, lazy_loads=lazy)
        for m, vl in ((None, None), (mask, valid)):
            md, vd = (None if m is None else E.to_device(m)), (None if vl is None else E.to_device(vl))
            want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125, mask=m, valid_len=vl)
            outs = []
            for mod in (E, variant):
                plain = mod.fused_attention(q, k, v, nn, bs, luts["blocks"], 0.125, mask=md, valid_len=vd).numpy()
                ws = zeros(E.schedule_workspace_bytes(sched, B, H, bs, d))
                cut = mod.fused_attention_scheduled(q, k, v, nn, items, sched, ws, bs, luts["blocks"], 0.125, mask=md,
                                                    valid_len=vd).numpy()
                outs.append((plain, cut))
            assert rel_err(outs[1][0], want) <= TOL[True] and rel_err(outs[1][1], want) <= TOL[True]
            assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])


def test_kernels_under_the_undefined_behaviour_sanitizer(E, request):
    """The host build compiled with -fsanitize=undefined in trapping mode (misaligned vector accesses, indices past
    fixed arrays, out-of-range shifts, signed overflow): one pass over the attention entry points.  A finding ends
    the process with an illegal-instruction trap, which is the failure.  Takes minutes to build: only with --ubsan."""
    if not request.config.getoption("--ubsan"):
        pytest.skip("needs --ubsan (a build of several minutes)")
    S = emu_lib.load("ubsan")
    for case in cases([(64, 64), (32, 96), (64, 40)]):
        if case[3] == 0:
            test_fused_forward_plain_scheduled_streamed(S, *case)
            test_fused_backward(S, *case)
    for bs, d in ((64, 64), (32, 120)):
        test_unfused_sequence_bf16(S, bs, d, 0, True)
    test_unfused_sequence_fp32(S, 64, 36)
    test_scheduled_launch_with_one_table_per_head(S)
    import scheduled_dsd_cases
    poisoned = lambda n: emu_lib.empty((max(int(n), 256),), torch.uint8, fill=0xFF)   # noqa: E731
    for bs, d, bf16, tables in ((64, 64, True, 1), (32, 40, True, 4), (64, 36, False, 1)):
        scheduled_dsd_cases.products(S, emu_lib.tensor, poisoned, bs, d, bf16, tables)


@pytest.mark.parametrize("name,args", [("attention_host_test", []),
                                       ("transformer_inference", ["2", "2", "256", "2", "64", "bf16"]),
                                       ("transformer_inference", ["1", "1", "256", "2", "64", "f32"])])
def test_cpp_host_programs_on_the_host_build(name, args):
    """The C++ mains of sf-bert_amd/host/ -- one in the shape of the reference's *_fusion_test.cu that goes through the
    reference-named launchers (bst_sgemm_nt, BlocksparseMaskedSoftmax, bst_sgemm_xn, fusion_attention2,
    fusion_attention) of the replacement headers, one in the shape of transformer_inference_part.cpp on
    sfb_model_forward -- compiled against the stand-in runtime and linked with the host build of the kernels."""
    import subprocess
    exe = emu_lib.build_host_program(name)
    out = subprocess.run([exe] + args, capture_output=True, text=True, timeout=900)
    assert out.returncode == 0 and "PASSED" in out.stdout, (out.stdout[-600:], out.stderr[-600:])
