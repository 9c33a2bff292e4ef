import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    """The opened GPU 0 through the C ABI. The HIP library must be there: a missing one is an error, not a skip."""
    from nextsycl_amd import Gpu, api

    a = api()
    if a.gpu_count() < 1:
        pytest.fail("no GPU visible to libnextsycl-llm.so")
    g = Gpu.open(0)
    yield g
    g.close()


@pytest.fixture
def tune(ops):
    """Sets the library's tuning knobs (ns_attn_tune) for one test; every knob touched goes back to 0 = the default."""
    touched = set()

    def set_knob(knob, value):
        touched.add(knob)
        ops.tune(knob, value)

    yield set_knob
    for k in touched:
        ops.tune(k, 0)


@pytest.fixture(scope="session")
def ops(gpu):
    from nextsycl_amd.attn import Ops

    return Ops(gpu)
