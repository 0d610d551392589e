import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _seed_per_test(request):
    """Every test draws the same random inputs whatever ran before it: the
    global generators (torch CPU and, lazily, GPU; numpy's legacy one) are
    seeded from the test's id."""
    import zlib

    import numpy as np
    import torch
    seed = zlib.crc32(request.node.nodeid.encode()) & 0x7FFFFFFF
    torch.manual_seed(seed)
    np.random.seed(seed)
    yield


@pytest.fixture(autouse=True)
def _reset_config():
    """Every test starts from the default global config."""
    from exact_amd.conf import QuantizationConfig, config
    fresh = QuantizationConfig()
    saved = dict(config.__dict__)
    config.__dict__.update(fresh.__dict__)
    yield
    config.__dict__.clear()
    config.__dict__.update(saved)


def _use_emulated_backend(monkeypatch):
    """Run the Python layers on CPU tensors against the SIMT-emulated build of
    the kernels (tests/emu): same .hip sources, same C ABI.  Only tests do
    this; the package itself has no CPU path."""
    import itertools

    import torch

    import emu_util
    from exact_amd import _lib
    from exact_amd.cpp_extension import _checks, quantization

    monkeypatch.setattr(_lib, "_lib", emu_util.emu())
    monkeypatch.setattr(_checks, "on_device", lambda t: True)
    monkeypatch.setattr(_checks, "stream_ptr", lambda t: None)
    counter = itertools.count(1)
    monkeypatch.setattr(quantization, "next_philox", lambda device: (0xC0FFEE, 4 * next(counter)))
    return torch.device("cpu")


@pytest.fixture(params=["emulated", pytest.param("gpu", marks=pytest.mark.gpu)])
def backend(request, monkeypatch):
    """Device on which a layer-level test runs: the real GPU (marked gpu) or
    CPU tensors over the emulated kernels."""
    import torch
    if request.param == "gpu":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        return torch.device("cuda:0")
    return _use_emulated_backend(monkeypatch)
