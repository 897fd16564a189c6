import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """The margin of the gradient comparisons of this run (tests/helpers.py: assert_gradients_close)."""
    try:
        from helpers import WORST_GRADIENT as w, GRAD_SUM_STEPS
    except Exception:
        return
    if w["elements"]:
        terminalreporter.write_line(
            f"gradients: {w['elements']} elements compared, {w['beyond_stated_bar']} beyond 1e-4 rel + 1e-6 abs alone; "
            f"worst error / bound {w['ratio']:.3f} ({w['where']}); rounding steps needed {w['needed_steps']:.2f} of {GRAD_SUM_STEPS:g} allowed")
