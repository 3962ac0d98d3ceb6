"""The library's kernels against the golden fixtures written by the reference's own CPU functions (golden_cases.py):
on the device (marked gpu), and from the same sources on the host model of the kernels (CPU suite)."""
import numpy as np
import pytest
import torch

import emu_lib
import golden_cases
from test_emulated_kernels import E   # noqa: F401  (fixture: the host build)


def device_backend():
    from sfb import sfb
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()   # noqa: E731
    zeros = lambda n: torch.zeros(max(int(n), 256), dtype=torch.uint8, device="cuda")   # noqa: E731
    return sfb, dev, zeros


def host_backend(E):
    emu_lib.configure()
    return E, emu_lib.tensor, lambda n: emu_lib.empty((max(int(n), 256),), torch.uint8, fill=0)


@pytest.mark.gpu
@pytest.mark.parametrize("fixture", golden_cases.FORWARD_FIXTURES)
def test_attention_forward_against_the_reference_outputs_on_the_device(fixture):
    golden_cases.attention_forward(*device_backend(), fixture=fixture)


@pytest.mark.gpu
@pytest.mark.parametrize("fixture", golden_cases.FORWARD_FIXTURES)
def test_attention_backward_against_the_reference_outputs_on_the_device(fixture):
    golden_cases.attention_backward(*device_backend(), fixture=fixture)


@pytest.mark.gpu
def test_layer_ops_and_loss_against_the_reference_outputs_on_the_device():
    S, dev, _ = device_backend()
    golden_cases.layer_ops(S, dev)
    golden_cases.cross_entropy(S, dev)


@pytest.mark.parametrize("fixture", golden_cases.FORWARD_FIXTURES)
def test_attention_forward_against_the_reference_outputs_on_the_host_model(E, fixture):
    golden_cases.attention_forward(*host_backend(E), fixture=fixture)


@pytest.mark.parametrize("fixture", golden_cases.FORWARD_FIXTURES)
def test_attention_backward_against_the_reference_outputs_on_the_host_model(E, fixture):
    golden_cases.attention_backward(*host_backend(E), fixture=fixture)


def test_layer_ops_and_loss_against_the_reference_outputs_on_the_host_model(E):
    S, dev, _ = host_backend(E)
    golden_cases.layer_ops(S, dev)
    golden_cases.cross_entropy(S, dev)
