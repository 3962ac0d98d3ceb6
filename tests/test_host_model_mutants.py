"""Do the tests on the host model notice mistakes in the real kernels?  Each case builds the host model with one
deliberate mistake in a kernel source -- a wait or a barrier taken out of a tile pipeline, a swizzle dropped on the
loading side, a merge that does not wait for its partial records, an arrival counter that is not reset, a counted wait
one tile short, chunk sums of a cut line that overwrite one another or are left out of the reduction -- and expects
the corresponding test of the CPU suite to FAIL under at least one of the lane orders / load timings it uses (and the
unmodified build to pass, which the CPU suite checks anyway).
A build per mistake: minutes.  Run with `pytest tests/test_host_model_mutants.py --mutants`."""
import pytest
import torch

import emu_lib
import test_emulated_kernels as T
from test_emulated_kernels import E   # noqa: F401  (fixture)

WAIT = "        do { emu::s_waitcnt_vmcnt(0); } while (0);\n        __syncthreads();\n    };"

MUTANTS = {
    "forward_tiles_read_without_the_wait": dict(
        source="fused_attention.hip", count=2, old=WAIT, new="        __syncthreads();\n    };"),
    "forward_tiles_read_without_the_barrier": dict(
        source="fused_attention.hip", count=2, old=WAIT, new="        do { emu::s_waitcnt_vmcnt(0); } while (0);\n    };"),
    "loader_without_the_swizzle": dict(
        source="tile_index.h", old="return rr * row_bytes + ((pos ^ swz(8u * odd + rr)) << 4);",
        new="return rr * row_bytes + (pos << 4);"),
    "backward_tiles_read_without_the_wait": dict(
        source="fused_backward.hip", count=2,
        old="            do { emu::s_waitcnt_vmcnt(0); } while (0);\n            __syncthreads();",
        new="            __syncthreads();"),
    "merge_does_not_wait_for_its_records": dict(
        source="fused_attention.hip", old="if (++polls > kMaxPolls) { ready = 0; break; }", new="break;"),
    "arrival_counter_not_reset": dict(
        source="fused_attention.hip",
        old="if (t == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);", new=";"),
    "dsd_wait_one_tile_short": dict(
        source="unfused_attention.hip", old="do { emu::s_waitcnt_vmcnt((0)); } while (0)",
        new="do { emu::s_waitcnt_vmcnt((DsdStreamWait::V_LOADS)); } while (0)"),
    "chunks_of_a_cut_line_share_a_record": dict(
        source="unfused_attention.hip", old="it.nchunks > 1 ? it.part + it.chunk + 1 : 0u", new="it.nchunks > 1 ? it.part + 1 : 0u"),
    "reduction_leaves_out_the_last_chunk": dict(
        source="unfused_attention.hip", old="for (uint32_t ch = 0; ch < it.nchunks; ++ch)\n            sum +=",
        new="for (uint32_t ch = 0; ch + 1 < it.nchunks; ++ch)\n            sum +="),
}


def scheduled_dsd(M, order, lazy):
    import scheduled_dsd_cases
    emu_lib.configure(order=order, lazy_loads=lazy)
    poisoned = lambda n: emu_lib.empty((max(int(n), 256),), torch.uint8, fill=0xFF)   # noqa: E731
    scheduled_dsd_cases.products(M, emu_lib.tensor, poisoned, 64, 64, True)


CHECKS = {
    "chunks_of_a_cut_line_share_a_record": scheduled_dsd,
    "reduction_leaves_out_the_last_chunk": scheduled_dsd,
    "forward_tiles_read_without_the_wait": lambda M, o, l: T.test_fused_forward_plain_scheduled_streamed(M, 64, 64, True, o, l),
    "forward_tiles_read_without_the_barrier": lambda M, o, l: T.test_fused_forward_plain_scheduled_streamed(M, 64, 64, True, o, l),
    "loader_without_the_swizzle": lambda M, o, l: T.test_fused_forward_plain_scheduled_streamed(M, 64, 64, True, o, l),
    "backward_tiles_read_without_the_wait": lambda M, o, l: T.test_fused_backward(M, 64, 64, True, o, l),
    "merge_does_not_wait_for_its_records": lambda M, o, l: T.test_fused_forward_plain_scheduled_streamed(M, 64, 64, True, o, l),
    "arrival_counter_not_reset": lambda M, o, l: T.test_fused_forward_plain_scheduled_streamed(M, 64, 64, True, o, l),
    "dsd_wait_one_tile_short": lambda M, o, l: T.test_unfused_sequence_bf16(M, 64, 64, o, l),
}


@pytest.mark.parametrize("name", sorted(MUTANTS))
def test_a_seeded_mistake_is_noticed(E, name, request):
    if not request.config.getoption("--mutants"):
        pytest.skip("needs --mutants (a build of the host model per mistake)")
    mutant = emu_lib.load("mutant_" + name, MUTANTS[name])
    noticed = []
    for order, lazy in T.MODES + [(33, True), (34, False), (35, True), (36, False)]:
        try:
            CHECKS[name](mutant, order, lazy)
        except (AssertionError, mutant.SfbError) as failure:
            noticed.append((order, lazy, str(failure)[:80]))
    print(name, "noticed under", [(o, l) for o, l, _ in noticed])
    assert noticed, "the mistake went unnoticed under every order and timing"


def test_a_merge_that_runs_out_of_its_wait_is_reported_and_the_workspace_recovers(E, request):
    """A merge that waits for a partial record nobody writes (the plan's copy on the device is altered: the merge of the
    last records expects one record more than exist, whose flag -- in the padding of the flag area -- is never set), in
    a build with a short bound on the wait (64 polls instead of 2^20): the merge gives up, the launch reports status
    1, nothing hangs and every other row is right; the binding then clears the workspace (sfb_stream_reset), and the
    next launch, with the plan as built, is right and reports 0."""
    if not request.config.getoption("--mutants"):
        pytest.skip("needs --mutants (a build of the host model)")
    import numpy as np
    import oracle_lib as orc
    short = emu_lib.load("mutant_short_merge_wait", dict(
        source="fused_attention.hip", old="constexpr uint32_t kMaxPolls = 1u << 20;", new="constexpr uint32_t kMaxPolls = 1u << 6;"))
    emu_lib.configure()
    bs, nb, B, H, d = 64, 5, 2, 2, 64
    luts = short.build_luts(T.layout(short, nb))   # two long rows per head: they are what the plan cuts
    Q, K, V = T.inputs(B, nb * bs, H, d, 77, True)
    q, k, v = (T.dev(x, True) for x in (Q, K, V))
    nn = short.to_device(luts["nn_lut"])
    stream = short.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=24, d=d, bf16=True, masked=False)
    n_parts = stream["plan"].n_parts
    assert n_parts > 0 and (4 * n_parts) % 256 != 0, "the flag area has padding after the last flag"
    ws = T.zeros(short.stream_workspace_bytes(stream, d))
    want = orc.attention(Q, K, V, luts["nn_lut"], bs, 0.125)
    good = stream["blob"].copy()
    merges = stream["merges"]
    last = int(np.argmax(merges["part"] + merges["nparts"]))
    assert merges["part"][last] + merges["nparts"][last] == n_parts
    merges["nparts"][last] += 1            # (a view of stream["blob"])
    starved = (int(merges["batch"][last]), int(merges["head"][last]), int(merges["row"][last]))
    out = short.fused_attention_streamed(q, k, v, nn, short.to_device(stream["blob"]), stream, ws, bs, luts["blocks"], 0.125,
                                         out=emu_lib.empty((B, nb * bs, H, d), torch.float32, fill=7.0)).numpy()
    assert short.stream_status(stream, d, ws) == 1          # (and the binding has reset the workspace)
    b, h, r = starved
    assert (out[b, r * bs:(r + 1) * bs, h] == 7.0).all(), "the starved row is left alone"
    out[b, r * bs:(r + 1) * bs, h] = want[b, r * bs:(r + 1) * bs, h]
    assert T.rel_err(out, want) <= T.TOL[True]
    for _ in range(2):
        got = short.fused_attention_streamed(q, k, v, nn, short.to_device(good), stream, ws, bs, luts["blocks"], 0.125)
        assert short.stream_status(stream, d, ws) == 0
        assert T.rel_err(got.numpy(), want) <= T.TOL[True]
