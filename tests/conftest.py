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


def pytest_terminal_summary(terminalreporter):
    """How far the gradient comparisons leaned on the rounding-noise allowance (helpers.NOISE_LOG), worst first."""
    try:
        import helpers
    except ImportError:
        return
    rows = [r for r in helpers.NOISE_LOG if r[2] or r[3]]
    if not rows:
        return
    rows.sort(key=lambda r: -(r[2] / max(r[1], 1)))
    terminalreporter.write_line("gradient comparisons that used the noise allowance: %d of %d tensors" % (
        len(rows), len(helpers.NOISE_LOG)))
    for name, size, noisy, loud in rows[:25]:
        terminalreporter.write_line("  %-40s %9d elements, %6d needed it (%.2g), %5d with a loud allowance" % (
            name, size, noisy, noisy / max(size, 1), loud))
