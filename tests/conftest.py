import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests", "golden")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _seed():
    np.random.seed(42)
    yield


def oracle_backend():
    """The CPU oracle as a ``configs.Backend`` (NumPy value type on the repo tracer)."""
    import autograd_amd as ag
    import oracle.anp as anp
    from autograd_amd import configs

    return configs.Backend(
        name="oracle (NumPy restatement)",
        np=anp,
        logsumexp=anp.logsumexp,
        grad=ag.grad,
        elementwise_grad=ag.elementwise_grad,
        make_hvp=ag.make_hvp,
        make_jvp=ag.make_jvp,
        put=lambda a: a,
        get=np.asarray,
        sync=lambda: None,
    )
