import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: test needs a real MI355X (run with -m gpu)')


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped (not failed) when no device is present, so an unfiltered
    ``pytest tests`` works in the build container; ``-m gpu`` on the GPU box runs them."""
    try:
        import torch

        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason='no GPU in this environment')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """How many compared entries met the pure relative bounds and how many needed the absolute floors."""
    try:
        from tolerances import FLOOR_STATS
    except Exception:
        return
    for kind, (total, pure, _) in FLOOR_STATS.items():
        if total:
            terminalreporter.write_line(
                f'parity bars, {kind}s: {total} entries compared, {100.0 * pure / total:.3f} % within the relative bound alone, '
                f'{total - pure} needed the absolute floor')
