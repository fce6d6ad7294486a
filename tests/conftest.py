import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu on the GPU box)')


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason='no GPU in this environment')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _library_heuristics_restored():
    """A test that pins a kernel variant or sets a tuning knob and then fails must not change what later tests run."""
    yield
    from dlblas_amd import _lib
    if _lib.loaded():
        _lib.force_variant(None)
        for knob in _lib.KNOBS:
            _lib.tune(knob, 0)


def pytest_terminal_summary(terminalreporter):
    """Relative error at the strict floor (|ref| floored at 1e-3 rms) of every parity check that ran: reported, not
    asserted (the asserted bars are in helpers.tolerance_check)."""
    try:
        import helpers
    except ImportError:
        return
    log = helpers.strict_floor_log
    if not log:
        return
    worst = sorted(log, key=lambda kv: -kv[1])[:12]
    terminalreporter.write_line(f'parity checks against the exact oracle: {len(log)}; largest relative errors at the 1e-3 rms floor:')
    for what, err in worst:
        terminalreporter.write_line(f'  {err:.3e}  {what}')
