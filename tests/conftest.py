import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__ as entry
    return entry.load_package()


@pytest.fixture(scope="session")
def gpu(pkg):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    pkg.check(pkg.lib().vx_init(0), "vx_init")
    return pkg


@pytest.fixture(scope="session")
def oracle():
    import reflib
    return reflib.load_oracle()


@pytest.fixture(scope="session")
def ref():
    import reflib
    r = reflib.load_ref()
    if r is None:
        pytest.skip("oracle/_ref (the reference's ggml-cpu) was not prebuilt")
    return r
