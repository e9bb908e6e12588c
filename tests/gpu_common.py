"""Fixtures shared by the GPU parity tests (all call through the C ABI)."""
import numpy as np
import pytest


@pytest.fixture(scope="module")
def backend():
    from slai_amd.runtime import Backend
    b = Backend(0)
    yield b
    b.close()


def rel_err(got, ref):
    """max-abs error relative to the largest reference magnitude (the bar for logits is 1e-2)."""
    return float(np.abs(np.asarray(got, np.float64) - np.asarray(ref, np.float64)).max() / max(np.abs(ref).max(), 1e-30))
