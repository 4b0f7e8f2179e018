"""pytest configuration: the `gpu` marker and helpers shared by the suites."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def mt19937_raw(seed, n):
    """First n 32-bit outputs of std::mt19937(seed) (init_genrand seeding)."""
    bg = np.random.MT19937()
    bg._legacy_seeding(int(seed))
    return bg.random_raw(n).astype(np.uint32)


@pytest.fixture
def rng():
    return np.random.default_rng(0x5EED)


@pytest.fixture
def tune(monkeypatch):
    """Tuning overrides of the kernel library (VLA_ATTN_*, VLA_GEMM_*, VLA_TERNARY_TILE).

    The library reads them from the environment once, never on a launch path, so a test that
    changes one asks it to read them again; everything is restored when the test ends."""
    from util import pkg

    class Tune:
        def set(self, key, value):
            monkeypatch.setenv(key, str(value))
            pkg.lib().vla_kernels_reload_env()

        def clear(self, *keys):
            for k in keys:
                monkeypatch.delenv(k, raising=False)
            pkg.lib().vla_kernels_reload_env()

    yield Tune()
    monkeypatch.undo()
    pkg.lib().vla_kernels_reload_env()
