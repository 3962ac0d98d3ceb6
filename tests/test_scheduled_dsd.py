"""The block-sparse x dense products launched over work items (scheduled_dsd_cases.py): on the device (marked gpu), and
from the same sources on the host model of the kernels (CPU suite), there also with the lanes taken in adverse orders."""
import numpy as np
import pytest
import torch

import emu_lib
import scheduled_dsd_cases as cases
from test_emulated_kernels import E   # noqa: F401  (fixture: the host build)

# block size, head size, bf16 operands, heads with a table of their own (1: one layout for all)
SHAPES = [(64, 64, True, 1), (64, 64, False, 1), (32, 64, True, 1), (32, 40, True, 1), (32, 96, False, 1),
          (64, 128, True, 1), (64, 64, True, 4), (64, 20, False, 4)]


def device_backend():
    from sfb import sfb
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()   # noqa: E731
    poisoned = lambda n: torch.full((max(int(n), 256),), 0xFF, dtype=torch.uint8, device="cuda")   # noqa: E731
    return sfb, dev, poisoned


def host_backend(E, **how):
    emu_lib.configure(**how)
    return E, emu_lib.tensor, lambda n: emu_lib.empty((max(int(n), 256),), torch.uint8, fill=0xFF)


@pytest.mark.gpu
@pytest.mark.parametrize("bs,d,bf16,tables", SHAPES)
def test_products_over_work_items_on_the_device(bs, d, bf16, tables):
    cases.products(*device_backend(), bs, d, bf16, tables)


@pytest.mark.gpu
def test_a_context_of_bigbird_length_cut_as_the_launch_suggests_on_the_device():
    # 64 block-rows, the global ones of 64 blocks: the shape the cut is for
    S, dev, poisoned = device_backend()
    cases.products(S, dev, poisoned, 64, 64, True, max_blocks=16, nb=64, B=1, H=2)


@pytest.mark.gpu
def test_argument_errors_on_the_device():
    cases.argument_errors(*device_backend())


@pytest.mark.parametrize("bs,d,bf16,tables", [SHAPES[0], SHAPES[4], SHAPES[7]])
def test_products_over_work_items_on_the_host_model(E, bs, d, bf16, tables):
    cases.products(*host_backend(E), bs, d, bf16, tables)


@pytest.mark.parametrize("order", [14, 21])
def test_products_over_work_items_with_lanes_in_adverse_orders(E, order):
    if order == 14:
        cases.products(*host_backend(E, order=order, lazy_loads=True), 64, 64, True, 1)
    else:
        cases.products(*host_backend(E, order=order, lazy_loads=False), 32, 40, True, 4)


def test_argument_errors_on_the_host_model(E):
    cases.argument_errors(*host_backend(E))
