import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def fwp():
    """The product package (its directory name is not a Python identifier)."""
    return importlib.import_module("recurrent-fwp_amd")


@pytest.fixture(params=["scan", "chunked", "split", "phase"])
def delta_kernels(request, fwp):
    """The kinds of delta-rule kernels for D = 16/32: the step-by-step scan, 16-step blocks on the
    matrix cores with one wave per sequence, those blocks split over several waves, and (16 x 16
    states) the blocks of a sequence prepared in parallel with a one-product chain.  The sum rule
    has the first two and, for states of more than one 16 x 16 tile, several waves per sequence under the
    last two; other shapes take the LDS kernels whatever the setting."""
    L_ = fwp._lib
    L_.config(L_.CFG_DELTA_KERNELS, {"scan": L_.DELTA_SCAN, "chunked": L_.DELTA_CHUNKED, "split": L_.DELTA_SPLIT,
                                      "phase": L_.DELTA_PHASE}[request.param])
    yield request.param
    L_.config(L_.CFG_DELTA_KERNELS, L_.DELTA_AUTO)
