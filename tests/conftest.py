"""Shared pytest setup: marker registration, import path, and numeric helpers.

CPU tests (`-m "not gpu"`) cover the oracle, the host logic and the exported
C-ABI symbol table. GPU tests (`-m gpu`) are the parity tests proper and call
the HIP kernels through the C-ABI of libvibevoice_hip.so.
"""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def scaled_rel_err(got, ref) -> float:
    """max|got-ref| / (max|ref| + 1e-9): the reference's own tolerance scale
    (tests/test_cpu_kernels.c:36-54)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if got.size == 0:
        return 0.0
    return float(np.max(np.abs(got - ref)) / (np.max(np.abs(ref)) + 1e-9))


def half_order(bits) -> np.ndarray:
    """Map FP16 bit patterns to integers whose difference counts FP16 steps
    (+0 and -0 coincide)."""
    b = np.asarray(bits, dtype=np.uint16).astype(np.int32)
    mag = b & 0x7FFF
    return np.where(b & 0x8000, -mag, mag)


def ulp16_diff(a_bits, b_bits) -> np.ndarray:
    return np.abs(half_order(a_bits) - half_order(b_bits))
