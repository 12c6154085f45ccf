import os
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = ROOT / "tests" / "golden" / "ql_goldens.npz"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import Oracle

    return Oracle()


@pytest.fixture(scope="session")
def ref():
    """The reference's own CPU kernels; only where oracle/_ref was built."""
    from oracle.binding import Ref

    if not Ref.available():
        pytest.skip("oracle/_ref not built on this machine (no reference tree)")
    return Ref()


@pytest.fixture(scope="session")
def golden():
    assert GOLDEN.exists(), "tests/golden/ql_goldens.npz is missing (tests/golden/make_goldens.py writes it)"
    return np.load(GOLDEN, allow_pickle=False)


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def capi():
    from llaminar_amd import capi as c

    c.load()  # raises if the HIP library is missing: GPU tests must not pass without it
    return c


def rel_err(y: np.ndarray, ref: np.ndarray) -> float:
    """max |y - ref| / max |ref|  (the bound the fp32 output contract is stated in)."""
    denom = float(np.abs(ref).max())
    if denom == 0.0:
        return float(np.abs(y).max())
    return float(np.abs(y.astype(np.float64) - ref.astype(np.float64)).max() / denom)
