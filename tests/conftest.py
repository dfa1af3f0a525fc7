import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """The worst logit error the model-level comparisons saw, as a part of the largest logit: the
    bfloat16 bound in replay_checks.py is set from this line."""
    try:
        from replay_checks import WORST
    except Exception:
        return
    if WORST:
        terminalreporter.write_line("worst logit error against the plain implementation, of the largest logit: " +
                                    ", ".join(f"{k} {v:.3e}" for k, v in sorted(WORST.items())))
