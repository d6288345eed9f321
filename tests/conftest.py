import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu")


@pytest.fixture(scope="session")
def oracle():
    from oracle import rans_oracle

    rans_oracle.build()
    return rans_oracle


@pytest.fixture
def always_fused(monkeypatch):
    """Many-row inputs normally decode the weight once and call a library GEMM; with this fixture they stay
    on the fused kernels (one decode per pass of rows)."""
    from comp_inference_amd import linear_hip, transposed_linear_hip

    monkeypatch.setattr(linear_hip, "DECODE_ONCE_ABOVE_ROWS", None)
    monkeypatch.setattr(transposed_linear_hip, "DECODE_ONCE_ABOVE_ROWS", None)
