import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box only)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure), compiled on demand with g++."""
    from oracle import binding
    binding.build()
    binding.lib()
    return binding


@pytest.fixture(scope="session")
def qm():
    """The product library binding; no fallback if it is not built."""
    import importlib
    return importlib.import_module("qingming-qwen3-tts_amd").binding


@pytest.fixture(scope="session")
def engine():
    """The engine-shell library binding (libqm_engine.so); no fallback if it is not built."""
    import importlib
    return importlib.import_module("qingming-qwen3-tts_amd.engine")


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")
