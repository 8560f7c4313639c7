"""Shared fixtures: the C ABI loader, the CPU oracle and seeded fp8 inputs."""
import importlib.util
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "tensor-core-fp8_amd")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_package():
    """Import the package directory (its name has a hyphen) as tensor_core_fp8_amd."""
    name = "tensor_core_fp8_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "__init__.py"))
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def load_oracle():
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle  # noqa: E402
    return oracle


@pytest.fixture(scope="session")
def pkg():
    return load_package()


@pytest.fixture(scope="session")
def oracle():
    return load_oracle()


def finite_codes(fmt):
    """All fp8 codes that decode to a finite number."""
    c = np.arange(256, dtype=np.uint8)
    if fmt == 0:
        return c[(c & 0x7F) != 0x7F]
    return c[((c >> 2) & 0x1F) != 0x1F]


def random_codes(rng, shape, fmt):
    """Uniform over the finite codes of the format (covers subnormals, extremes, -0)."""
    pool = finite_codes(fmt)
    return pool[rng.integers(0, pool.size, size=shape)]
