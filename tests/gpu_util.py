"""Helpers shared by the GPU parity tests."""
import numpy as np
import pytest

import tract_amd


@pytest.fixture(scope="session")
def rt():
    return tract_amd.runtime_for_name("rocm")


def max_abs(a, b):
    return float(np.abs(np.asarray(a, dtype=np.float64) - np.asarray(b, dtype=np.float64)).max())
