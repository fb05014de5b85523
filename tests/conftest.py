import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.oracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    """The real vecops CPU matmul, where oracle/_ref was built and the host has AMX."""
    from oracle.oracle import Reference
    ref = Reference.load()
    if ref is None:
        pytest.skip("oracle/_ref/libvecops_ref.so not built or host lacks AMX")
    return ref


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    """max |got - want| / max(1, |want|, |got|): the scaling of the reference's own
    conversion checks (tests/ops/MatmulConversionTestCommon.h:72-85)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    if got.size == 0:
        return 0.0
    scale = np.maximum(1.0, np.maximum(np.abs(got), np.abs(want)))
    return float((np.abs(got - want) / scale).max())
