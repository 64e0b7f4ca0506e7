import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import pyoracle
    return pyoracle.oracle()


@pytest.fixture(scope="session")
def reference():
    from oracle import pyoracle
    ref = pyoracle.reference()
    if ref is None:
        pytest.skip("oracle/_ref/libmako_ref.so not built (needs /root/reference)")
    return ref


@pytest.fixture(scope="session")
def gpu_ctx():
    from mako_amd import hip
    from mako_amd.api import SamplerContext
    if hip.device_count() < 1:
        pytest.fail("no HIP device: GPU tests need an MI355X")
    hip.set_device(0)
    ctx = SamplerContext(max_rows=256, max_vocab=151552, max_hist=4096)
    yield ctx
    ctx.close()
