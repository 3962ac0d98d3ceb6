"""bench.py run end to end without a GPU: the library is the host build of the kernels (tests/emu_lib.py), every timed
loop runs its body once and clocks are fakes.  What this checks is the script itself -- that every leg still calls the
binding the way the binding wants to be called and that the one JSON line carries what its readers expect -- not a
number: the figures in the line are meaningless here."""
import json
import sys

import pytest
import torch

import emu_lib


class FakeEvent:
    def __init__(self, enable_timing=False):
        pass

    def record(self, stream=None):
        pass

    def elapsed_time(self, other):
        return 1.0


@pytest.mark.parametrize("workload", ["c1"])
def test_bench_line_of_the_smallest_workload(workload, capsys):
    import bench
    with pytest.MonkeyPatch.context() as patch:
        mod = emu_lib.install(patch)
        emu_lib.configure()
        patch.setitem(sys.modules, "sf-bert_amd", mod)
        patch.setattr(torch.cuda, "is_available", lambda: True)
        patch.setattr(torch.cuda, "Event", FakeEvent)
        patch.setattr(torch.cuda, "empty_cache", lambda: None)

        def once(torch_, fn, *a, **k):
            fn()
            return 1.0
        patch.setattr(bench, "_time", once)
        patch.setattr(bench, "_median_ms", once)
        patch.setattr(bench, "RAMP_SECONDS", 0.0)
        patch.setattr(sys, "argv", ["bench.py", "--workload", workload, "--steps", "1", "--warmup", "0"])
        bench.main()
    lines = [ln for ln in capsys.readouterr().out.splitlines() if ln.startswith("{")]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 1 and line["vs_baseline"] is None and line["data"] == "synthetic"
    assert "workload" in line["config"] and "model" not in line["config"]
    roof = line["roofline"]
    assert roof["bound"] in ("mfma", "hbm") and roof["unit"] in ("TFLOP/s", "GB/s")
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-12 and "traffic" in roof
    cpu = line["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    for leg in ("streamed", "unfused", "dsd_scheduled", "backward_unfused", "backward_fused", "cpu_reference_single_thread"):
        assert leg in line and "error" not in line[leg], (leg, line[leg])


def test_layer_and_model_legs_at_a_small_shape():
    """The two legs that only the full-size workload runs, called with their shape shrunk."""
    import bench
    with pytest.MonkeyPatch.context() as patch:
        mod = emu_lib.install(patch)
        emu_lib.configure()
        patch.setattr(torch.cuda, "Event", FakeEvent)
        patch.setattr(torch.cuda, "empty_cache", lambda: None)

        def once(torch_, fn, *a, **k):
            fn()
            return 1.0
        patch.setattr(bench, "_time", once)
        bs, H, d, nb = 64, 2, 64, 4
        patch.setattr(bench, "LAYER_SHAPE", {"B": 1, "L": nb * bs, "ffn": 256, "vocab": 512, "layers": 2})
        luts = mod.build_luts(bench.make_layout(mod, "bigbird", nb))
        layer = bench.time_layer(mod, torch, luts, bs, H, d, 2)
        assert layer["ms_per_layer_bf16"] == 1.0 and layer["ms_per_layer_f32"] == 1.0
        assert layer["roofline_bf16"]["peak"] == bench.PEAK_TFLOPS["bf16"]
        model = bench.time_model(mod, torch, luts, bs, H, d, 2)
        # a freshly initialised model predicts uniformly: loss = ln(vocabulary), up to the spread of the random logits
        for name in ("bf16", "f32"):
            assert abs(model["loss_" + name] - 6.238) < 0.1, model


def test_smoke_entry_on_the_host_build(capsys):
    """__graft_entry__.smoke() with the library replaced by the host build of its sources."""
    import __graft_entry__ as entry
    with pytest.MonkeyPatch.context() as patch:
        mod = emu_lib.install(patch)
        emu_lib.configure()
        patch.setitem(sys.modules, "sf-bert_amd", mod)
        patch.setattr(torch.cuda, "is_available", lambda: True)
        entry.smoke()
    assert capsys.readouterr().out.count("max rel err") == 2
