"""Helpers shared by the GPU parity tests."""
import numpy as np
import pytest

from cnet_amd import capi, ops


@pytest.fixture(scope="session")
def gpu():
    capi.init(0)
    yield capi.device_info()


def rel(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def rel_c(got, want):
    """relative Frobenius error of a complex quantity given as (re, im) pairs"""
    g = np.asarray(got[0], np.float64) + 1j * np.asarray(got[1], np.float64)
    w = np.asarray(want[0], np.float64) + 1j * np.asarray(want[1], np.float64)
    return float(np.linalg.norm(g - w) / max(np.linalg.norm(w), 1e-30))


def seeded(port, seed, shape, sig=1.0):
    return port.normal(seed, shape, 0.0, sig)


# The parity bar of this build: relative Frobenius error of every output and Wirtinger gradient against the CPU path.
TOL = 1e-4
