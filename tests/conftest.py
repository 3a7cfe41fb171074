import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped when no GPU is visible, so that a plain
    `pytest tests/` on a CPU box stays green."""
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(params=["groups", "by_row"])
def pair_form(request, monkeypatch):
    """Runs a test once with the rule books in their grouped form only and once with the pairs also
    kept by stationary row, which makes the convolution take its by-row kernel whatever the density."""
    from sphconv_amd import rulebook
    if request.param == "by_row":
        monkeypatch.setattr(rulebook, "BY_ROW_MIN_PAIRS", 0.0)
    else:
        monkeypatch.setattr(rulebook, "BY_ROW_MIN_PAIRS", float("inf"))
    return request.param
