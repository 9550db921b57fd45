import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

os.environ.setdefault("BACKEND", "hip")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ops():
    """(hip_op, oracle_op) lookup through the registry, the way the reference compares two backends
    (mops/registry.py:32-36)."""
    from nano_vllm_ninetoothed_amd import mops
    import oracle.mops_torch  # noqa: F401  registers the "torch" backend

    def pair(name):
        return mops.get_op(name, "hip"), mops.get_op(name, "torch")

    return pair


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran without a GPU")
    from nano_vllm_ninetoothed_amd import _capi

    _capi.load()  # the hip extension must be present: there is no fallback to hide behind
    return torch.device("cuda:0")
