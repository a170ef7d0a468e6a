import importlib
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def from_bits(a):
    """numpy array from a golden file -> torch tensor (uint16 arrays are bf16 bit patterns)."""
    a = np.asarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return torch.from_numpy(a.copy())


def bits_equal(a, b):
    """bit-for-bit equality of two bf16 (or any same-dtype) tensors."""
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    if a.dtype == torch.bfloat16:
        return torch.equal(a.contiguous().view(torch.int16), b.contiguous().view(torch.int16))
    return torch.equal(a, b)


def bf16_ulp_diff(a, b):
    """distance in bf16 units-in-the-last-place between two bf16 tensors (monotone integer map)."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return (key(a) - key(b)).abs()


@pytest.fixture(scope="session")
def hyc():
    """the product package (its directory name is not a Python identifier)."""
    return importlib.import_module("hyc-lora_amd")


@pytest.fixture(scope="session")
def golden_compress():
    return np.load(os.path.join(GOLDEN, "compress_cases.npz"))


@pytest.fixture(scope="session")
def golden_softmax():
    return np.load(os.path.join(GOLDEN, "softmax_cases.npz"))


@pytest.fixture(scope="session")
def golden_modules():
    return np.load(os.path.join(GOLDEN, "module_cases.npz"))
