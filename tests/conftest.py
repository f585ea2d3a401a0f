import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


def bf16_bits(x_f32: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even."""
    from oracle import mlx_affine as o

    return o.f32_to_bf16_bits(np.asarray(x_f32, dtype=np.float32))


from cases import seeded  # noqa: E402,F401  (kept importable from conftest)


@pytest.fixture(scope="session")
def oracle():
    from oracle import mlx_affine as o

    o.clib()
    return o
