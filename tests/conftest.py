import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# `kernel` is imported by bare name, exactly as the reference's model.py does (inference/model.py:13-15)
for p in (ROOT, os.path.join(ROOT, "zk-deepseek_amd"), os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as ora
    return ora


@pytest.fixture(scope="session")
def zk_tables():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "zk_tables.json")) as f:
        return json.load(f)


@pytest.fixture(autouse=True)
def _library_switches_at_their_defaults():
    """a test that forces a GEMM path or lets softmax clobber its input must not decide what the next test runs on,
    whatever the order: both switches are back at their defaults before every test (once the library is loaded)"""
    k = sys.modules.get("kernel")
    if k is not None and hasattr(k, "lib"):
        k.lib.zk_gemm_set_path(0)
        k.lib.zk_softmax_clobber_input(0)
    yield
