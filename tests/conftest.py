import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:  # pragma: no cover
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def single_rank_by_default(request):
    """Every GPU test starts from a world of one rank, whatever the test before it set up (the tests that play one
    rank of a grid call initialize(...) themselves)."""
    if "gpu" in request.keywords:
        from cubework_amd.distributed import initialize
        initialize(None, 1)
    yield


@pytest.fixture
def oracle64():
    """The oracle evaluates its formulas in float64 for the duration of the test."""
    import torch
    import oracle
    with oracle.precision(torch.float64):
        yield


def pytest_terminal_summary(terminalreporter, exitstatus, config):
    """Achieved parity errors of the session: the ten comparisons closest to their bar, and the whole list
    in $CW_PARITY_LOG when that names a file."""
    try:
        from tests.util import PARITY_LOG
    except Exception:  # pragma: no cover
        return
    if not PARITY_LOG:
        return
    path = os.environ.get("CW_PARITY_LOG")
    if path:
        with open(path, "w") as f:
            f.write("what\tdtype\terr\tbar\n")
            for what, dt, err, tol in PARITY_LOG:
                f.write("%s\t%s\t%.3e\t%.1e\n" % (what, dt, err, tol))
    worst = sorted(PARITY_LOG, key=lambda r: -(r[2] / r[3] if r[3] > 0 else 0.0))[:10]
    terminalreporter.write_line("parity: %d comparisons; closest to their bar:" % len(PARITY_LOG))
    for what, dt, err, tol in worst:
        terminalreporter.write_line("  %-60s %-9s err %.2e  bar %.1e" % (what[:60], dt, err, tol))
