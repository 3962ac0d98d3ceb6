"""The host model of the kernels (tests/emu_lib.py, tests/emu/) checked on itself: its matrix instruction against
numpy, and that it notices the mistakes it is there to notice -- an LDS-direct load read without a wait, LDS data of
another wave read without a barrier, a buffer refilled while it is still read -- under at least one of the lane orders
and load timings the tests use, while the correct forms pass under all of them."""
import ctypes as C

import numpy as np
import pytest

import emu_lib

ORDERS = [0, 1, 7, 14, 21]   # ascending, descending, shuffled (these also hold waves back at random)


@pytest.fixture(scope="module")
def lib():
    mod = emu_lib.load()
    yield mod.lib
    emu_lib.configure()


def buffers():
    src = np.random.default_rng(1).integers(0, 255, 4096, dtype=np.uint8)   # 255 never occurs: unwritten LDS is 0xff
    dst = np.zeros(2048, np.uint8)
    return src, dst


def ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def exchange(lib, wait, barrier, order, lazy):
    emu_lib.configure(order=order, lazy_loads=lazy)
    src, dst = buffers()
    assert lib.emu_selftest_exchange(ptr(src), ptr(dst), wait, barrier) == 0, emu_lib.message()
    return bool((dst == src[:2048]).all())


def test_correct_exchange_passes_under_every_order_and_timing(lib):
    for order in ORDERS:
        for lazy in (True, False):
            assert exchange(lib, 1, 1, order, lazy)


def test_a_missing_wait_is_noticed_when_loads_land_late(lib):
    assert not any(exchange(lib, 0, 1, order, True) for order in ORDERS)
    # (with loads that land at once the mistake is invisible: the two timings are both needed)
    assert all(exchange(lib, 0, 1, order, False) for order in ORDERS)


def test_a_missing_barrier_is_noticed(lib):
    assert not all(exchange(lib, 1, 0, order, lazy) for order in ORDERS for lazy in (True, False))


def refill(lib, barrier, order, lazy):
    emu_lib.configure(order=order, lazy_loads=lazy)
    src, dst = buffers()
    assert lib.emu_selftest_refill(ptr(src), ptr(dst), barrier) == 0, emu_lib.message()
    return bool((dst[:1024] == src[1024:2048]).all() and (dst[1024:] == src[2048:3072]).all())


def test_a_buffer_refilled_while_it_is_read(lib):
    for order in ORDERS:
        for lazy in (True, False):
            assert refill(lib, 1, order, lazy)
    assert not all(refill(lib, 0, order, lazy) for order in ORDERS for lazy in (True, False))


def test_matrix_instruction_against_numpy(lib):
    emu_lib.configure()
    rng = np.random.default_rng(2)
    a = rng.standard_normal((32, 16)).astype(np.float32)
    b = rng.standard_normal((16, 32)).astype(np.float32)
    a16 = (a.view(np.uint32) >> 16).astype(np.uint16)   # truncation: exact bf16 values
    b16 = (b.view(np.uint32) >> 16).astype(np.uint16)
    at = (a16.astype(np.uint32) << 16).view(np.float32)
    bt = (b16.astype(np.uint32) << 16).view(np.float32)
    d = np.zeros((32, 32), np.float32)
    assert lib.emu_selftest_mfma(ptr(a16), ptr(b16), ptr(d)) == 0, emu_lib.message()
    want = at.astype(np.float64) @ bt.astype(np.float64)
    assert np.abs(d - want).max() <= 1e-5
    # an asymmetric case: one nonzero in A and B each, so a transposed operand or result cannot pass
    a16[:], b16[:] = 0, 0
    a16[5, 11], b16[11, 20] = 0x4000, 0x4040   # 2.0, 3.0
    assert lib.emu_selftest_mfma(ptr(a16), ptr(b16), ptr(d)) == 0
    assert d[5, 20] == 6.0 and np.count_nonzero(d) == 1


def test_wave_wide_operation_under_divergence(lib):
    emu_lib.configure()
    lib.emu_reset_counts()
    out = np.zeros(64, np.uint32)
    assert lib.emu_selftest_diverged(ptr(out)) == 0, emu_lib.message()
    want = 1000 + np.arange(64)
    want[8:32] = 1008   # the first active lane's value
    assert (out == want).all()
    assert emu_lib.counts()["readfirstlane"][1] >= 1   # counted as executed with part of the wave
