import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped (not failed) when no device is visible, so that a plain
    `pytest tests/` on a CPU-only machine stays green."""
    have_gpu = None
    for item in items:
        if "gpu" in item.keywords:
            if have_gpu is None:
                try:
                    import torch

                    have_gpu = torch.cuda.is_available()
                except Exception:
                    have_gpu = False
            if not have_gpu:
                item.add_marker(pytest.mark.skip(reason="no GPU visible"))


def pytest_terminal_summary(terminalreporter):
    """Parity figures of the GPU tests: one line per comparison against the oracle."""
    try:
        import gpu_harness
    except Exception:
        return
    if gpu_harness.PARITY_LOG:
        terminalreporter.section("attention parity against the oracle (unscaled contract figures)")
        for line in gpu_harness.PARITY_LOG:
            terminalreporter.write_line(line)
