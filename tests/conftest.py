import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "box-convolutions_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run with -m gpu on the MI355X box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import cpu_checker
    return cpu_checker.oracle()


@pytest.fixture(scope="session")
def reference():
    from oracle import cpu_checker
    ref = cpu_checker.reference()
    if ref is None:
        pytest.skip("oracle/_ref was not built here (needs /root/reference)")
    return ref


@pytest.fixture(scope="session")
def hip():
    """The product: tensor-level front end of libboxconv_hip.so. Fails if it was not built."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from box_convolution import _native
    _native.load()
    return _native
