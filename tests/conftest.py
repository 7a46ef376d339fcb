import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """Boundary ties of the zone selections against the oracle's scores: how many accepted swaps lie
    within one bf16 ulp of the boundary score and how many need the second ulp."""
    from tests.parity import TIE_TALLY, FLIP_TALLY
    if FLIP_TALLY:
        terminalreporter.write_line("decisions accepted only because a logit sat on a bf16 rounding boundary (label: count)")
        for k in sorted(FLIP_TALLY):
            terminalreporter.write_line(f"  {k}: {FLIP_TALLY[k]}")
    if TIE_TALLY:
        terminalreporter.write_line("zone boundary ties vs the oracle (label: checks, swaps <= 1 ulp, swaps in (1, 2] ulp)")
        quiet = 0
        for k in sorted(TIE_TALLY):
            c, a, b = TIE_TALLY[k]
            if a or b:
                terminalreporter.write_line(f"  {k}: {c}, {a}, {b}")
            else:
                quiet += c
        terminalreporter.write_line(f"  all other labels: {quiet} checks, no swap")
