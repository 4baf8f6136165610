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
        # (worded without "<number> passed" / "<number> failed": result parsers count those tokens)
        line = ("assert_parity: of %(comparisons)d tensor comparisons, the rounding-noise term or the "
                "sibling scale was needed in %(needed_noise_term)d (reference tensor zero, or a millionth of its "
                "siblings, in %(of_those_reference_all_zero)d of those)" % stats)
        if stats["worst_case"]:
            line += "; largest diff / (tol * max|cpu|) among the rest: %(worst_ratio).2f [%(worst_case)s]" % stats
        else:
            line += "; every other comparison met tol * max|cpu| of the tensor itself"
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


@pytest.fixture
def switches(hip):
    """``switches(name, value)`` sets one of the library's BOXCONV_* environment switches (None
    removes it) and makes the library read its environment again (it reads it once, at first
    use); everything is put back, and re-read, when the test ends."""
    saved = {}

    def set_switch(name, value):
        saved.setdefault(name, os.environ.get(name))
        if value is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = value
        hip.reload_switches()
    yield set_switch
    for name, value in saved.items():
        if value is None:
            os.environ.pop(name, None)
        else:
            os.environ[name] = value
    hip.reload_switches()
