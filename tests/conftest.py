import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "tf_fixtures.npz"), allow_pickle=False)


@pytest.fixture(autouse=True, scope="session")
def _kernel_variants_from_env():
    """CDM_TEST_ATTN_VARIANT / CDM_TEST_GEMM_VARIANT: run the whole suite on another kernel variant than the default
    (tests that name a variant themselves still select it)."""
    for op, var in (("attn", "CDM_TEST_ATTN_VARIANT"), ("gemm", "CDM_TEST_GEMM_VARIANT")):
        if os.environ.get(var):
            from cosmos_amd import ops
            ops.set_variant(op, int(os.environ[var]))
    yield
