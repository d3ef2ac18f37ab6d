import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_c():
    from oracle import akv_oracle_c
    akv_oracle_c.build()
    return akv_oracle_c


def pytest_terminal_summary(terminalreporter):
    from tests.common import WORST_STEP_ERR
    if WORST_STEP_ERR:
        terminalreporter.write_line("worst max-abs error of attention outputs against the oracle, per comparison site:")
        for k in sorted(WORST_STEP_ERR):
            terminalreporter.write_line(f"  {WORST_STEP_ERR[k]:.3e}  {k}")
