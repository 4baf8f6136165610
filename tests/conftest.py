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


def pytest_terminal_summary(terminalreporter):
    stats = getattr(sys.modules.get("test_gpu_parity"), "NOISE_STATS", None)
    if stats and stats["comparisons"]:
        line = ("assert_parity: %(comparisons)d tensor comparisons, %(needed_noise_term)d passed only with the "
                "rounding-noise term or the sibling scale (%(of_those_reference_all_zero)d of those have an "
                "all-zero reference tensor)" % stats)
        terminalreporter.write_line(line)
        path = os.environ.get("BOXCONV_PARITY_REPORT")
        if path:
            with open(path, "a") as fh:
                fh.write(line + "\n")


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
