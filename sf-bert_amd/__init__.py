"""sf-bert_amd: MI355X-native block-sparse attention path of SF-BERT.

Python host mirror of the C ABI in include/sfbert_hip.h (ctypes; torch tensors are used only as
device buffers and for the current stream).  Import with importlib.import_module("sf-bert_amd").
The HIP library is mandatory: there is no CPU or PyTorch fallback.
"""
from .capi import *  # noqa: F401,F403
from . import capi  # noqa: F401
