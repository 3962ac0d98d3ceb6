"""Do the tests on the host model notice mistakes in the real kernels?  Each case builds the host model with one
deliberate mistake in a kernel source -- a wait or a barrier taken out of a tile pipeline, a swizzle dropped on the
loading side, a merge that does not wait for its partial records, an arrival counter that is not reset, a counted wait
one tile short -- and expects the corresponding test of test_emulated_kernels.py to FAIL under at least one of the
lane orders / load timings it uses (and the unmodified build to pass, which the CPU suite checks anyway).
A build per mistake: minutes.  Run with `pytest tests/test_host_model_mutants.py --mutants`."""
import pytest

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
}

CHECKS = {
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
