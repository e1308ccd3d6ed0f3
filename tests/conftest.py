"""Shared test plumbing: paths, the `gpu` marker and small helpers."""
import importlib.util
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
PACKAGE = ROOT / "cpu-llms-in-c_amd"
for extra in (PACKAGE, ROOT / "oracle", ROOT):
    if str(extra) not in sys.path:
        sys.path.insert(0, str(extra))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as module  # oracle/oracle.py
    module.lib()
    return module


@pytest.fixture(scope="session")
def engine():
    import mi355q  # cpu-llms-in-c_amd/mi355q.py
    mi355q.library()
    return mi355q


@pytest.fixture(scope="session")
def gpu(engine):
    """One engine context on GPU 0 for the whole session; fails loudly without one."""
    context = engine.Context(0)
    yield context
    context.close()


@pytest.fixture
def force(gpu):
    """force(name, value): sets an experiment knob of the shared context (launch shape, kernel
    variant) for the duration of one test."""
    names = []

    def apply(name, value):
        gpu.set_option(name, value)
        names.append(name)

    yield apply
    for name in names:
        gpu.set_option(name, None)


def q4_relative_error(y, reference):
    """max_i |y_i - ref_i| / max(|ref_i|, 1e-2 * rms(ref)), per activation row."""
    y = np.asarray(y, dtype=np.float64)
    reference = np.asarray(reference, dtype=np.float64)
    worst = 0.0
    for row, ref_row in zip(y.reshape(-1, y.shape[-1]), reference.reshape(-1, y.shape[-1])):
        rms = float(np.sqrt(np.mean(ref_row * ref_row)))
        floor = max(1e-2 * rms, 1e-30)
        worst = max(worst, float(np.max(np.abs(row - ref_row) / np.maximum(np.abs(ref_row), floor))))
    return worst


def bf16_bits(values):
    """fp32 -> bf16 bits, round to nearest even (numpy integer restatement)."""
    bits = np.asarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = bits + 0x7FFF + ((bits >> 16) & 1)
    return ((bits >> 16) & 0xFFFF).astype(np.uint16)


def bf16_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
