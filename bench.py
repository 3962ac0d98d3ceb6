"""Benchmark of the fused block-sparse attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c3|c2|c1] [--dtype bf16|f32]

One step = one fused attention call over the whole batch of the workload (default: the BigBird
configuration B4 H12 L4096 d64 block 64, bf16 inputs, fp32 accumulation and output).  Inputs are
synthetic N(0,1) tensors already resident in HBM when the timed region starts.  Prints ONE JSON line:
metric/value = effective TFLOP/s over the nonzero blocks (nnz*B*H*4*bs^2*d flops per call), plus
`roofline` (MFMA bound, measured with HIP events on the launch stream), `cpu_baseline` (the CPU
oracle timed on this host's cores on a bounded sample of the same workload) and
`cpu_reference_single_thread` (the reference's own CPU attention functions, one thread as the reference is
built, at the smallest configuration's shape).
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}   # MI355X dense MFMA peaks
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (pattern, B, H, L, d, bs, default dtype)
    "c1": ("local", 1, 12, 512, 64, 32, "f32"),
    "c2": ("fixed", 8, 12, 1024, 64, 32, "f32"),
    "c3": ("strided", 8, 12, 2048, 64, 64, "bf16"),
    "c4": ("bigbird", 4, 12, 4096, 64, 64, "bf16"),
}


def make_layout(sfb, pattern, nb):
    if pattern == "local":
        return sfb.layout_local(nb, 1, bidirectional=True)
    if pattern == "fixed":
        return sfb.layout_fixed(1, nb, 4, causal=False)[0]
    if pattern == "strided":
        return sfb.layout_strided(nb, 4, 4)
    return sfb.layout_bigbird(nb, 1, 2, True, sfb.bigbird_draw(nb, 1, 2, True, 3, 1234))


def cpu_reference_single_thread():
    """The reference's CPU attention as it is built (one thread, dense L x L buffers, causal: transformer.cpp:533-545)
    at the shape of the smallest configuration, B1 H12 L512 d64: the reference's own functions compiled into
    oracle/_ref where that library exists, otherwise the oracle's block loops on one thread over the same causal
    layout."""
    import numpy as np
    import oracle_lib as orc
    B, H, L, d, bs = 1, 12, 512, 64, 32
    Q, K, V = (orc.fill_normal((B, L, H, d), 910 + i) for i in range(3))
    scale = 1.0 / np.sqrt(d)
    flops = 4.0 * B * H * (L * (L + 1) / 2) * d      # useful multiply-adds of the causal triangle
    if orc.ref is not None:
        from test_oracle_attention import ref_dense_causal
        run, kind = (lambda: ref_dense_causal(Q, K, V, scale)), "reference"
    else:
        from test_oracle_attention import causal_case
        _, _, _, luts, words = causal_case(B, H, L, d, bs, seed=910)
        run, kind = (lambda: orc.attention(Q, K, V, luts["nn_lut"], bs, scale, mask=words, nthreads=1)), "port"
    run()
    times = []
    t_begin = time.perf_counter()
    while len(times) < 10 and time.perf_counter() - t_begin < 5.0:
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    dt = sum(times) / len(times)
    return {"ms_per_call": dt * 1e3, "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": kind,
            "sample": "dense causal attention B1 H12 L512 d64 fp32, %d calls" % len(times)}


def cpu_baseline(luts, B, H, L, d, bs, bf16, flops):
    """Times the CPU oracle (a port of the reference CPU path) on the whole workload, repeated until
    about ten seconds of wall time have been spent on this host's cores."""
    import numpy as np
    import oracle_lib as orc
    threads = max(1, min(16, os.cpu_count() or 1))
    Q, K, V = (orc.fill_normal((B, L, H, d), 900 + i) for i in range(3))
    if bf16:
        Q, K, V = (orc.round_bf16(x) for x in (Q, K, V))
    times = []
    t_begin = time.perf_counter()
    while len(times) < 30 and time.perf_counter() - t_begin < 10.0:
        t0 = time.perf_counter()
        orc.attention(Q, K, V, luts["nn_lut"], bs, 1.0 / np.sqrt(d), nthreads=threads)
        times.append(time.perf_counter() - t0)
    dt = sum(times) / len(times)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "CPU oracle (fp32 port of the matmul.h/ewops.h loops over nonzero blocks, OpenMP over "
                      "block-rows) on the full workload, %d calls, mean %.3f s per call" % (len(times), dt),
            "ms_per_call": dt * 1e3}


def read_traffic(workload, dtype):
    """HBM bytes per launch of the fused kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and
    scaled by a plain copy kernel; recorded in profiles/ (null when no measurement is on file)."""
    path = os.path.join(ROOT, "profiles", "fused_attention_%s_%s_hbm_traffic.txt" % (workload, dtype))
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return float(line.split(":")[1])
    except OSError:
        pass
    return None


RAMP_SECONDS, RAMP_BATCH = 0.3, 200   # untimed launches before the warm-up steps


def _time(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def _median_ms(torch, fn, groups=40, per_group=50):
    """Median over groups of back-to-back launches (one event pair per group, so the events' own cost and the gaps
    they open between launches stay out of the figure)."""
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(groups)]
    for a, b in pairs:
        a.record()
        for _ in range(per_group):
            fn()
        b.record()
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) / per_group for a, b in pairs)
    return times[len(times) // 2]


def time_streamed(sfb, torch, luts, q, k, v, bs, blocks, scale, flops, peak):
    """The same attention launched over streams (resident work-groups walking chained items, sfb_build_stream):
    few long chunks of the cut rows, no dynamic tail."""
    B, L, H, d = q.shape
    stream = sfb.build_stream(luts["nn_lut"], L // bs, B, H, bs, level=False)
    blob = sfb.to_device(stream["blob"])
    ws = torch.zeros(sfb.stream_workspace_bytes(stream, d), dtype=torch.uint8, device="cuda")
    out = torch.empty((B, L, H, d), device="cuda", dtype=torch.float32)
    nn = sfb.to_device(luts["nn_lut"])
    fn = lambda: sfb.fused_attention_streamed(q, k, v, nn, blob, stream, ws, bs, blocks, scale, out=out)
    ms = _time(torch, fn, 500, 100)
    assert sfb.stream_status(stream, d, ws) == 0
    return {"ms_per_call": ms, "frac_of_mfma_peak": flops / (ms * 1e-3) / 1e12 / peak, "streams": int(stream["plan"].wg_slots),
            "partial_records": int(stream["plan"].n_parts), "balance": float(stream["plan"].balance)}


def time_unfused(sfb, torch, luts, q, k, v, bs, blocks, scale, bf16, fused_ms):
    """sdd -> masked softmax -> dsd with S and P in HBM (bf16 storage for bf16 inputs, else fp32)."""
    B, L, H, d = q.shape
    nb = L // bs
    store = torch.bfloat16 if bf16 else torch.float32
    nt, nn = sfb.to_device(luts["nt_lut"]), sfb.to_device(luts["nn_lut"])
    S = torch.empty((B, H, blocks, bs, bs), device="cuda", dtype=store)
    P = torch.empty_like(S)
    O = torch.empty((B, L, H, d), device="cuda", dtype=torch.float32)

    def trio():
        sfb.bst_sgemm_nt(nt, q, k, bs, blocks, c=S)
        sfb.BlocksparseMaskedSoftmax(nn, None, S, nb, scale, y=P)
        sfb.bst_sgemm_xn(nn, P, v, nb, c=O)

    ms = _time(torch, trio, 200, 50)
    parts = {"sdd_ms": _time(torch, lambda: sfb.bst_sgemm_nt(nt, q, k, bs, blocks, c=S), 200, 20),
             "softmax_ms": _time(torch, lambda: sfb.BlocksparseMaskedSoftmax(nn, None, S, nb, scale, y=P), 200, 20),
             "dsd_ms": _time(torch, lambda: sfb.bst_sgemm_xn(nn, P, v, nb, c=O), 200, 20)}
    # HBM rate of each stage on its algorithmic bytes: the sparse tensor once, the dense operands / result once
    sparse_bytes = S.numel() * S.element_size()
    dense_bytes = q.numel() * q.element_size()
    parts["sdd_hbm_GBs"] = (2 * dense_bytes + sparse_bytes) / parts["sdd_ms"] / 1e6
    parts["softmax_hbm_GBs"] = 2 * sparse_bytes / parts["softmax_ms"] / 1e6
    parts["dsd_hbm_GBs"] = (sparse_bytes + dense_bytes + O.numel() * 4) / parts["dsd_ms"] / 1e6
    # sdd + softmax in one kernel (P still goes through HBM): one work-group per block-row against the
    # reference's own decomposition, one work-group per block with flag / spin exchange
    order = sfb.to_device(luts["row_order"])
    parts["sdd_softmax_row_owner_ms"] = _time(
        torch, lambda: sfb.fusion_attention2(nn, q, k, bs, blocks, scale, y=P, row_order=order), 200, 20)
    nbytes = int(sfb.lib.sfb_split_softmax_scratch_bytes(bs, blocks, B, H, nb))
    scratch = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    status = []

    def split():
        status[:] = [sfb.fusion_attention2_split(nt, nn, q, k, bs, blocks, scale, y=P, scratch=scratch)[1]]
    parts["sdd_softmax_per_block_with_flags_ms"] = _time(torch, split, 100, 10)
    parts["sdd_softmax_per_block_status"] = int(status[0])
    return dict(ms_per_call=ms, fused_speedup=ms / fused_ms, sp_storage="bf16" if bf16 else "f32", **parts)


def time_dsd_scheduled(sfb, torch, luts, q, v, bs, blocks, bf16, max_blocks=16):
    """The two dsd products (P V over block-rows, P^T dO over block-columns) launched over work items of at most
    max_blocks blocks against the launch by lines, each with its HBM rate on the algorithmic bytes."""
    B, L, H, d = q.shape
    nb = L // bs
    store = torch.bfloat16 if bf16 else torch.float32
    P = torch.randn((B, H, blocks, bs, bs), device="cuda").to(store)
    c = torch.empty((B, L, H, d), device="cuda", dtype=torch.float32)
    moved = P.numel() * P.element_size() + v.numel() * v.element_size() + c.numel() * 4
    out = {"max_blocks": max_blocks}
    for name, key, op in (("nn", "nn_lut", sfb.NN_OP), ("tn", "tn_lut", sfb.TN_OP)):
        lut = sfb.to_device(luts[key])
        sched = sfb.build_schedule(luts[key], nb, max_blocks)
        items = sfb.to_device(sched["items"])
        ws = torch.empty(max(sfb.dsd_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
        by_items = _time(torch, lambda: sfb.bst_sgemm_xn_scheduled(lut, P, v, nb, items, sched, ws, op=op, c=c), 200, 20)
        by_lines = _time(torch, lambda: sfb.bst_sgemm_xn(lut, P, v, nb, op=op, c=c), 200, 20)
        out.update({name + "_items": sched["n_items"], name + "_cut_lines_parts": sched["n_parts"],
                    name + "_ms": by_items, name + "_hbm_GBs": moved / by_items / 1e6,
                    name + "_by_lines_ms": by_lines, name + "_by_lines_hbm_GBs": moved / by_lines / 1e6})
    return out


def time_backward(sfb, torch, luts, q, k, v, bs, blocks, scale, bf16):
    """Backward of the unfused path from the stored P (dV, dP, dS, dK, dQ), each stage and the whole chain, with
    the HBM rate of the two memory-bound stage types on their algorithmic bytes."""
    B, L, H, d = q.shape
    nb = L // bs
    code = sfb.BF16 if bf16 else sfb.F32
    ld = {name: sfb.to_device(luts[name]) for name in ("nt_lut", "nn_lut", "tn_lut")}
    p = sfb.fusion_attention2(ld["nn_lut"], q, k, bs, blocks, scale, out_dtype=code)
    d_out = torch.randn((B, L, H, d), device="cuda").to(q.dtype)
    dp, ds = torch.empty_like(p), torch.empty_like(p)
    c = torch.empty((B, L, H, d), device="cuda", dtype=torch.float32)
    sparse_bytes = p.numel() * p.element_size()
    dense_bytes = q.numel() * q.element_size()
    tn = _time(torch, lambda: sfb.bst_sgemm_xn(ld["tn_lut"], p, d_out, nb, op=sfb.TN_OP, c=c), 200, 20)
    grad = _time(torch, lambda: sfb.BlocksparseMaskedSoftmaxGrad(ld["nn_lut"], dp, p, nb, scale, dx=ds), 200, 20)
    o = sfb.bst_sgemm_xn(ld["nn_lut"], p, v, nb)
    delta = sfb.row_dot(d_out, o)
    schedules = sfb.dsd_schedules(luts, nb, B, H, bs, d)
    return {"ms_per_call": _time(torch, lambda: sfb.attention_backward(q, k, v, d_out, p, ld, bs, blocks, scale), 100, 20),
            "ms_per_call_products_over_work_items": _time(
                torch, lambda: sfb.attention_backward(q, k, v, d_out, p, ld, bs, blocks, scale, o=o, schedules=schedules), 100, 20),
            "ms_per_call_with_forward_output": _time(
                torch, lambda: sfb.attention_backward(q, k, v, d_out, p, ld, bs, blocks, scale, o=o), 100, 20),
            "row_dot_ms": _time(torch, lambda: sfb.row_dot(d_out, o), 200, 20),
            "sdd_softmax_grad_ms": _time(
                torch, lambda: sfb.sdd_softmax_grad(ld["nt_lut"], d_out, v, p, delta, bs, blocks, scale, ds=ds), 200, 20),
            "dsd_tn_ms": tn, "dsd_tn_hbm_GBs": (sparse_bytes + dense_bytes + c.numel() * 4) / tn / 1e6,
            "sdd_nt_ms": _time(torch, lambda: sfb.bst_sgemm_nt(ld["nt_lut"], d_out, v, bs, blocks, c=dp), 200, 20),
            "softmax_grad_ms": grad, "softmax_grad_hbm_GBs": 3 * sparse_bytes / grad / 1e6,
            "dsd_nn_ms": _time(torch, lambda: sfb.bst_sgemm_xn(ld["nn_lut"], ds, k, nb, c=c), 200, 20),
            "sp_storage": "bf16" if bf16 else "f32"}


def time_fused_backward(sfb, torch, luts, q, k, v, bs, blocks, scale, max_blocks, flops_forward):
    """Training pair of the fused path: forward with log-sum-exp output, then dQ, dK, dV in two kernels that keep
    P, dP and dS on chip.  Backward FLOPs counted as 2.5 x forward (five block products instead of two)."""
    B, L, H, d = q.shape
    nb = L // bs
    sched = sfb.build_schedule(luts["nn_lut"], nb, max_blocks)
    ws = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256), dtype=torch.uint8, device="cuda")
    nn, tn, items = sfb.to_device(luts["nn_lut"]), sfb.to_device(luts["tn_lut"]), sfb.to_device(sched["items"])
    d_out = torch.randn((B, L, H, d), device="cuda").to(q.dtype)
    fwd = lambda: sfb.fused_attention_forward_lse(q, k, v, nn, items, sched, ws, bs, blocks, scale)
    o, lse = fwd()
    rs, cs = sched, sfb.build_schedule(luts["tn_lut"], nb, max_blocks)
    rs["items_dev"], cs["items_dev"] = items, sfb.to_device(cs["items"])
    nbytes = int(sfb.lib.sfb_backward_workspace_bytes(rs["n_parts"], cs["n_parts"], B, H, bs, d))
    bws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device="cuda")
    bwd = lambda: sfb.fused_attention_backward(q, k, v, o, d_out, lse, nn, tn, bs, blocks, scale, row_sched=rs,
                                               col_sched=cs, workspace=bws)
    ms_b = _time(torch, bwd, 200, 20)
    return {"forward_with_lse_ms": _time(torch, fwd, 200, 20), "backward_ms": ms_b,
            "backward_TFLOPs": 2.5 * flops_forward / (ms_b * 1e-3) / 1e12}


GEMM_TUNING = 0   # what --gemm-tuning asked for (reported with the layer's numbers)
# shape of the encoder-layer and whole-model legs (BERT-base at the length of workload c4)
LAYER_SHAPE = {"B": 8, "L": 4096, "ffn": 3072, "vocab": 30522, "layers": 12}


def time_layer(sfb, torch, luts, bs, H, d, max_blocks, dtypes=("bf16", "f32"), steps=20):
    """One BERT-base encoder layer forward (hidden 768, FFN 3072, BigBird attention) at B8 L4096."""
    B, L, ffn, vocab = (LAYER_SHAPE[x] for x in ("B", "L", "ffn", "vocab"))
    n = H * d
    torch.manual_seed(1)
    w = {}
    for name, shape in (("wq", (n, n)), ("wk", (n, n)), ("wv", (n, n)), ("wo", (n, n)), ("w1", (n, ffn)),
                        ("w2", (ffn, n))):
        w[name] = torch.randn(shape, device="cuda") * 0.02
    for name, size in (("bq", n), ("bk", n), ("bv", n), ("bo", n), ("b1", ffn), ("b2", n), ("ln1_b", n),
                       ("ln2_b", n)):
        w[name] = torch.zeros(size, device="cuda")
    w["ln1_g"] = torch.ones(n, device="cuda")
    w["ln2_g"] = torch.ones(n, device="cuda")
    ids = torch.randint(0, vocab, (B, L), device="cuda", dtype=torch.int32)
    tok = torch.randn((vocab, n), device="cuda") * 0.02
    pos = torch.randn((L, n), device="cuda") * 0.02
    x = sfb.embedding_lookup(tok, ids, pos).reshape(B * L, n)
    out = {"shape": "B%d L%d hidden %d heads %d ffn %d, BigBird block %d" % (B, L, n, H, ffn, bs),
           "gemm_flops": 2.0 * B * L * (4 * n * n + 2 * n * ffn)}
    out["gemm_tuning"] = GEMM_TUNING
    y = torch.empty_like(x)
    attn_flops = luts["blocks"] * B * H * 4.0 * bs * bs * d
    for name, code in (("bf16", sfb.BF16), ("f32", sfb.F32)):
        if name not in dtypes:
            continue
        layer = sfb.EncoderLayer(w, luts, bs, H, d, ffn, dtype=code, max_blocks=max_blocks)
        ms = _time(torch, lambda: layer.forward(x, B, L, out=y), steps, 5)
        out["ms_per_layer_" + name] = ms
        # the layer's matrix work (GEMMs + attention blocks) against the MFMA peak of its operand type
        out["roofline_" + name] = {"bound": "mfma", "achieved": (out["gemm_flops"] + attn_flops) / (ms * 1e-3) / 1e12,
                                   "peak": PEAK_TFLOPS[name], "unit": "TFLOP/s",
                                   "frac": (out["gemm_flops"] + attn_flops) / (ms * 1e-3) / 1e12 / PEAK_TFLOPS[name]}
        assert torch.isfinite(y).all()
        del layer
    return out


def time_model(sfb, torch, luts, bs, H, d, max_blocks):
    """Forward pass of a whole BERT-base sized model (12 layers, hidden 768, FFN 3072, BigBird attention) with
    tied-embedding logits and cross-entropy loss over a 30522-token vocabulary at B8 L4096."""
    B, L, ffn, vocab, n_layers = (LAYER_SHAPE[x] for x in ("B", "L", "ffn", "vocab", "layers"))
    n = H * d
    torch.manual_seed(2)
    layers = []
    for _ in range(n_layers):
        w = {}
        for name, shape in (("wq", (n, n)), ("wk", (n, n)), ("wv", (n, n)), ("wo", (n, n)), ("w1", (n, ffn)),
                            ("w2", (ffn, n))):
            w[name] = torch.randn(shape, device="cuda") * 0.02
        for name, size in (("bq", n), ("bk", n), ("bv", n), ("bo", n), ("b1", ffn), ("b2", n), ("ln1_b", n),
                           ("ln2_b", n)):
            w[name] = torch.zeros(size, device="cuda")
        w["ln1_g"] = torch.ones(n, device="cuda")
        w["ln2_g"] = torch.ones(n, device="cuda")
        layers.append(w)
    tok = torch.randn((vocab, n), device="cuda") * 0.02
    pos = torch.randn((L, n), device="cuda") * 0.02
    ids = torch.randint(0, vocab, (B, L), device="cuda", dtype=torch.int32)
    labels = torch.randint(0, vocab, (B * L,), device="cuda", dtype=torch.int32)
    out = {"shape": "B%d L%d, %d layers hidden %d heads %d ffn %d, BigBird block %d, vocab %d, post-LN"
                    % (B, L, n_layers, n, H, ffn, bs, vocab),
           "gemm_flops": 2.0 * B * L * (n_layers * (4 * n * n + 2 * n * ffn) + n * vocab)}
    for name, code in (("bf16", sfb.BF16), ("f32", sfb.F32)):
        model = sfb.Model(tok, pos, layers, luts, bs, H, d, ffn, dtype=code, max_blocks=max_blocks, pre_ln=False)
        res = {}

        def step():
            res.update(model.forward(ids, labels))
        out["ms_per_forward_" + name] = _time(torch, step, 5, 2)
        out["loss_" + name] = float(res["loss"])
        del model
        torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default=None, choices=["bf16", "f32"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (reference kernel for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--layer-only", action="store_true",
                    help="only the bf16 encoder layer at B8 L4096, 200 timed calls (for a kernel trace of the layer)")
    ap.add_argument("--skip-extras", action="store_true",
                    help="only the fused-attention line: no unfused comparison, no encoder-layer timing")
    ap.add_argument("--gemm-tuning", type=int, default=0, choices=[0, 1],
                    help="how the GEMM seam picks its kernels (sfb_gemm_tuning): 0 = the library's short list, "
                         "1 = every kernel of the library that supports the problem (seconds per shape, once)")
    ap.add_argument("--heavy", type=int, default=-1,
                    help="override the schedule's number of leading items launched for all heads first")
    ap.add_argument("--max-blocks", type=int, default=-1,
                    help="split block-rows longer than this many key blocks (0 = one work-group per row, "
                         "-1 = what sfb_suggest_max_blocks gives for the launch's batch x heads)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path shards over (batch, head) with no exchange and "
              "this build has no multi-GPU leg; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    sfb = importlib.import_module("sf-bert_amd")
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(1)

    global GEMM_TUNING
    GEMM_TUNING = args.gemm_tuning
    sfb.gemm_tuning(args.gemm_tuning)
    pattern, B, H, L, d, bs, default_dtype = WORKLOADS[args.workload]
    dtype = args.dtype or default_dtype
    bf16 = dtype == "bf16"
    nb = L // bs
    luts = sfb.build_luts(make_layout(sfb, pattern, nb))
    blocks = luts["blocks"]
    if args.layer_only:
        layer_blocks = sfb.suggest_max_blocks(luts["nn_lut"], nb, 8 * H)
        print(json.dumps({"encoder_layer": time_layer(sfb, torch, luts, bs, H, d, layer_blocks, dtypes=("bf16",),
                                                      steps=200)}))
        return
    flops_per_bh = blocks * 4.0 * bs * bs * d
    flops = flops_per_bh * B * H
    elem = 2 if bf16 else 4
    algo_bytes = B * L * H * d * (3 * elem + 4)

    torch.manual_seed(0)
    tdt = torch.bfloat16 if bf16 else torch.float32
    q, k, v = (torch.randn((B, L, H, d), device="cuda", dtype=torch.float32).to(tdt) for _ in range(3))
    out = torch.empty((B, L, H, d), device="cuda", dtype=torch.float32)
    nn_lut = sfb.to_device(luts["nn_lut"])
    order = sfb.to_device(luts["row_order"])
    scale = 1.0 / (d ** 0.5)

    auto_blocks = args.max_blocks < 0
    if auto_blocks:
        args.max_blocks = sfb.suggest_max_blocks(luts["nn_lut"], nb, B * H)
    if args.max_blocks > 0:
        sched = sfb.build_schedule(luts["nn_lut"], nb, args.max_blocks)
        if args.heavy >= 0:
            sched["n_heavy"] = min(args.heavy, sched["n_items"] - 1)
        items = sfb.to_device(sched["items"])
        workspace = torch.zeros(max(sfb.schedule_workspace_bytes(sched, B, H, bs, d), 256),
                                dtype=torch.uint8, device="cuda")

        def step():
            sfb.fused_attention_scheduled(q, k, v, nn_lut, items, sched, workspace, bs, blocks, scale, out=out)
    else:
        def step():
            sfb.fused_attention(q, k, v, nn_lut, bs, blocks, scale, row_order=order, out=out)

    if args.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    # untimed: bring the clocks up before the warm-up steps (a handful of 50 us launches does not)
    ramp_until = time.perf_counter() + RAMP_SECONDS
    while time.perf_counter() < ramp_until:
        for _ in range(RAMP_BATCH):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    kernel_ms = start.elapsed_time(stop) / args.steps   # HIP events on the launch stream
    ms_per_step = wall_ms / args.steps
    assert torch.isfinite(out).all()
    median_ms = _median_ms(torch, step)

    traffic = read_traffic(args.workload, dtype)
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[dtype]
    result = {
        "metric": "fused block-sparse attn effective TFLOP/s + ms/layer at L=4096, 1 MI355X",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": "%s: %s block-sparse attention B%d H%d L%d d%d block %d, %d nonzero "
                               "blocks, %s inputs, fp32 accumulate/output" %
                               (args.workload, pattern, B, H, L, d, bs, blocks, dtype),
                   "max_blocks": args.max_blocks},
        "ms_per_attention_call": kernel_ms, "ms_per_attention_call_median": median_ms,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                     "frac": achieved / peak, "traffic": traffic,
                     "kernel": "fused_attention_%s_kernel<%d,%d>" % (dtype if bf16 else "f32", bs, d),
                     "algorithmic_flops_per_launch": flops, "avg_launch_ms": kernel_ms, "median_launch_ms": median_ms,
                     "frac_at_median": flops / (median_ms * 1e-3) / 1e12 / peak,
                     "hbm_algorithmic_bytes_per_launch": algo_bytes,
                     "hbm_achieved_GBs": algo_bytes / (kernel_ms * 1e-3) / 1e9,
                     "hbm_frac": algo_bytes / (kernel_ms * 1e-3) / 1e9 / PEAK_HBM_GBS},
    }
    def extra(name, fn, *fn_args):
        # the comparison legs are reported beside the metric; one of them failing must not cost the line
        try:
            result[name] = fn(*fn_args)
        except Exception as exc:   # noqa: BLE001 -- reported, not swallowed
            result[name] = {"error": "%s: %s" % (type(exc).__name__, exc)}
            print("bench.py: %s failed: %r" % (name, exc), file=sys.stderr)

    if not args.skip_extras:
        if bf16 or d == 64:
            extra("streamed", time_streamed, sfb, torch, luts, q, k, v, bs, blocks, scale, flops, peak)
        extra("unfused", time_unfused, sfb, torch, luts, q, k, v, bs, blocks, scale, bf16, kernel_ms)
        extra("dsd_scheduled", time_dsd_scheduled, sfb, torch, luts, q, v, bs, blocks, bf16)
        extra("backward_unfused", time_backward, sfb, torch, luts, q, k, v, bs, blocks, scale, bf16)
        extra("backward_fused", time_fused_backward, sfb, torch, luts, q, k, v, bs, blocks, scale, args.max_blocks, flops)
        if args.workload == "c4":
            # the layer and the model run eight sequences: their own chunk length
            layer_blocks = sfb.suggest_max_blocks(luts["nn_lut"], nb, 8 * H) if auto_blocks else args.max_blocks
            extra("encoder_layer", time_layer, sfb, torch, luts, bs, H, d, layer_blocks)
            extra("model_forward", time_model, sfb, torch, luts, bs, H, d, layer_blocks)
    if not args.no_cpu_baseline:
        extra("cpu_baseline", cpu_baseline, luts, B, H, L, d, bs, bf16, flops)
        extra("cpu_reference_single_thread", cpu_reference_single_thread)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
