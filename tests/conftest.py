import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def _oracle_lib():
    """The C oracle is test infrastructure: build it on demand (gcc only, a second)."""
    so = os.path.join(ROOT, "oracle", "libqfa_oracle.so")
    if not os.path.exists(so):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    yield


@pytest.fixture(scope="session")
def qfa():
    """The product package; on a GPU box a missing libqfa.so is an error, never a skip."""
    import quant_flash_attn_amd
    from quant_flash_attn_amd import _lib
    _lib.lib()
    return quant_flash_attn_amd
