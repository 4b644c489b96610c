import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP GPU (run on the MI355X box)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no HIP GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc
    orc.build()
    return orc


def pytest_terminal_summary(terminalreporter):
    """The values checks that came closest to their bound, and the largest relative errors seen."""
    try:
        from helpers import CHECK_LOG
    except Exception:
        return
    if not CHECK_LOG:
        return
    tr = terminalreporter
    tr.write_line(f"values checks: {len(CHECK_LOG)}; closest to their bound:")
    for what, ratio, rel, rtol in sorted(CHECK_LOG, key=lambda r: -r[1])[:8]:
        tr.write_line(f"  {what:<44s} |err|/bound {ratio:6.3f}   worst relative error {rel:.2e}   rtol {rtol:g}")
