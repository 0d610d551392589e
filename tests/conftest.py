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
def _reset_config():
    """Every test starts from the default global config."""
    from exact_amd.conf import QuantizationConfig, config
    fresh = QuantizationConfig()
    saved = dict(config.__dict__)
    config.__dict__.update(fresh.__dict__)
    yield
    config.__dict__.clear()
    config.__dict__.update(saved)
