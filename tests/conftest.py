import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (built on first use with gcc)."""
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def dmoe():
    """The HIP library through its C ABI; fails loudly when it is missing or no gfx950 is visible."""
    import torch
    from dmlx_amd import capi
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    capi.init(0)
    return capi


@pytest.fixture()
def ws(dmoe):
    w = dmoe.Workspace()
    yield w
    w.close()
