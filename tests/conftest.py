import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "diff-surfel-tracing_amd"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import surfel_oracle
    surfel_oracle.lib()  # builds with the committed Makefile if the .so is absent
    return surfel_oracle


@pytest.fixture(scope="session")
def tracer():
    """One SurfelTracer for the whole GPU session (the context owns grow-only BVH buffers)."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    import diff_surfel_tracing as dst
    return dst.SurfelTracer()
