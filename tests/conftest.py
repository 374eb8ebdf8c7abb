"""Shared fixtures. `-m "not gpu"` covers the oracle, the host encoder/policy and the C ABI's symbols on the CPU;
`-m gpu` tests are the parity tests proper: they call the HIP kernels through the C ABI and check them against the
oracle (oracle/, test infrastructure only)."""
from __future__ import annotations

import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import pyoracle

    pyoracle.lib()
    return pyoracle


@pytest.fixture(scope="session")
def ops():
    """The operator layer with the device initialised; fails (does not skip) when the HIP library is missing."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from orin_qwen_lossless_amd import ops as o

    o.init()
    return o


def golden(name: str):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    return z


def golden_names():
    return sorted(f[:-4] for f in os.listdir(GOLDEN) if f.endswith(".npz") and f != "cfg1_lut.npz")


# FP32 reassociation bound of the GEMV kernels relative to sum |w x| (reference tests/conftest.py:53-55)
GEMV_REL = 1e-5
BF16_REL = 2.0 ** -8
