import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box only)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "int8_conv_golden.npz")
    return dict(np.load(path, allow_pickle=False))


@pytest.fixture(scope="session")
def tie_golden():
    """Layer results on the one value where the reference's two rounding primitives differ (cases.TIE_ROUTE_CASES),
    written by the compiled reference through tests/golden/make_tie_route_golden.py."""
    path = os.path.join(ROOT, "tests", "golden", "tie_route_golden.npz")
    return dict(np.load(path, allow_pickle=False))


@pytest.fixture(scope="session")
def ref():
    """The compiled reference, where oracle/_ref/libotter_ref.so exists; otherwise the test is skipped."""
    from oracle.binding import Ref, ref_available
    if not ref_available():
        pytest.skip("oracle/_ref/libotter_ref.so not built (needs /root/reference)")
    return Ref()


@pytest.fixture(scope="session")
def hip():
    """The GPU library through its C ABI. Fails loudly if it is not built or no GPU is present."""
    import tensor_amd
    return tensor_amd.capi.Library()
