import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run on the MI355X box)")


def _gpu_available():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import shift_oracle
    shift_oracle.build()
    return shift_oracle.get()


@pytest.fixture(scope="session")
def ref_cpu_kernel():
    """The reference's own CPU kernel (oracle/_ref), or skip when it has not been built."""
    from oracle import shift_oracle
    mod = shift_oracle.load_reference_cpu_kernel()
    if mod is None:
        pytest.skip("oracle/_ref is not built (reference checkout absent)")
    return mod


@pytest.fixture
def rng():
    return np.random.default_rng(1234)


def random_codes(rng, shape, max_s=15, zero_frac=0.0, min_s=0):
    """Random right-shift amounts in [min_s, max_s] and signs in {-1,+1} (0 with prob zero_frac)."""
    s = rng.integers(min_s, max_s + 1, size=shape).astype(np.int32)
    sign = rng.choice(np.array([-1, 1], np.int32), size=shape)
    if zero_frac > 0:
        sign = np.where(rng.random(shape) < zero_frac, 0, sign).astype(np.int32)
    return s, sign


def random_activations(rng, shape, kind="mixed"):
    """int32 fixed-point activations: 'mixed' spans the whole 16.16 range incl. extremes."""
    if kind == "nonneg":
        return rng.integers(0, 2 ** 31 - 65536, size=shape).astype(np.int32)
    if kind == "small":
        return rng.integers(-(2 ** 20), 2 ** 20, size=shape).astype(np.int32)
    x = rng.integers(-(2 ** 31), 2 ** 31 - 1, size=shape, dtype=np.int64)
    flat = x.reshape(-1)
    extremes = np.array([0, 1, -1, 2 ** 31 - 1, -(2 ** 31), 2147418112, 65536, -65537], np.int64)
    n = min(flat.size, extremes.size)
    flat[:n] = extremes[:n]
    return x.astype(np.int32)


class Tune:
    """Forces a launch variant of the compute entry points through the library's test hook
    (``ds_test_tune``): ``Tune(planes=1, split=0)``, ``Tune(tile="4x16", split=4)``, ``Tune(cu=8)``."""

    def __init__(self, **knobs):
        self.knobs = {}
        for name, value in knobs.items():
            if value is None:
                continue
            if name == "tile":
                r, j = str(value).split("x")
                value = int(r) * 100 + int(j)
            self.knobs[name] = int(value)

    def __enter__(self):
        from deepshift_amd import _lib
        _lib.call("ds_test_tune", None, 0)
        for name, value in self.knobs.items():
            _lib.call("ds_test_tune", name.encode(), value)
        return self

    def __exit__(self, *exc):
        from deepshift_amd import _lib
        _lib.call("ds_test_tune", None, 0)
        return False
