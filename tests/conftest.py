import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def rel_err(a, b):
    """max|a-b| / max|b| with float64 accumulation (the parity metric)."""
    import torch
    a = a.detach().double().cpu() if not a.is_complex() else torch.view_as_real(a.detach().cpu().resolve_conj()).double()
    b = b.detach().double().cpu() if not b.is_complex() else torch.view_as_real(b.detach().cpu().resolve_conj()).double()
    denom = b.abs().max().item()
    if denom == 0.0:
        return (a - b).abs().max().item()
    return (a - b).abs().max().item() / denom
