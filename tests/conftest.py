import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "starrygl-framework_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    return o.load()[0]


@pytest.fixture(scope="session")
def oracle_cdll():
    from oracle import oracle as o
    return o.load()[1]


@pytest.fixture(scope="session")
def hot():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from starrygl_amd.lib import hot_path
    return hot_path("cuda:0")
